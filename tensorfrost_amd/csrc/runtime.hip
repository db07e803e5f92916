// Device lifetime, memory, hiprtc kernel cache, launch and timing for libtfhip.so.
//
// Plays the part that the OpenGL objects play for the reference's GPU backend
// (TensorFrost/Backend/Backends/OpenGL/{OpenGL.cpp,KernelManager.h,Memory.h}) and that
// g++/dlopen plays for its CPU backend (Backends/CPU/KernelCompiler.cpp): one device, one in-order
// stream, word-addressed buffers, source-in / launchable-handle-out.

#include <dlfcn.h>
#include <hip/hiprtc.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <condition_variable>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "common.h"

struct tfhip_kernel {
	hipModule_t module = nullptr;
	hipFunction_t function = nullptr;
	std::string name;
	bool owns_module = true;
};

struct tfhip_event {
	hipEvent_t ev = nullptr;
};

struct tfhip_graph {
	hipGraph_t graph = nullptr;
	hipGraphExec_t exec = nullptr;
	// Argument blocks of the module launches recorded into the graph: kept until the graph is destroyed.
	std::vector<std::unique_ptr<unsigned char[]>> arguments;
};

namespace tfhip {

static thread_local std::string g_last_error;

State& state() {
	static State s;
	return s;
}

int fail(int code, const char* fmt, ...) {
	char buf[2048];
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(buf, sizeof(buf), fmt, ap);
	va_end(ap);
	g_last_error = buf;
	return code;
}

int fail_hip(hipError_t err, const char* what) {
	return fail(TFHIP_ERR_HIP, "%s failed: %s (%s)", what, hipGetErrorName(err), hipGetErrorString(err));
}

void* scratch(size_t bytes) {
	State& s = state();
	if (bytes <= s.scratch_bytes) return s.scratch;
	if (s.capturing) {
		// Work already recorded points at the current scratch buffer.
		fail(TFHIP_ERR_STATE, "the scratch buffer would have to grow to %zu bytes while a graph is being recorded; run the same work once before recording", bytes);
		return nullptr;
	}
	if (s.scratch && s.live_graphs > 0) {
		// A recorded graph may carry this address in its kernel arguments: it stays valid until the last graph is gone.
		if (s.retired_scratch_count == sizeof(s.retired_scratch) / sizeof(s.retired_scratch[0])) {
			fail(TFHIP_ERR_STATE, "the scratch buffer had to grow more than %zu times while recorded graphs are alive; destroy graphs that are no longer needed",
			     s.retired_scratch_count);
			return nullptr;
		}
		s.retired_scratch[s.retired_scratch_count++] = s.scratch;
		s.scratch = nullptr;
		s.scratch_bytes = 0;
	}
	// The stream is in-order, but a kernel still reading the old scratch may be in flight.
	if (s.scratch) {
		hipStreamSynchronize(s.stream);
		hipFree(s.scratch);
		s.scratch = nullptr;
		s.scratch_bytes = 0;
	}
	size_t want = (bytes + 0xFFFFF) & ~size_t(0xFFFFF);  // 1 MiB granules
	hipError_t e = hipMalloc(&s.scratch, want);
	if (e != hipSuccess) {
		fail_hip(e, "hipMalloc(scratch)");
		return nullptr;
	}
	s.scratch_bytes = want;
	return s.scratch;
}

int check_async_error() {
	State& s = state();
	if (!s.async_error_host) return TFHIP_OK;
	const uint32_t code = *s.async_error_host;
	if (code == 0) return TFHIP_OK;
	*s.async_error_host = 0;
	return fail(TFHIP_ERR_HIP, "a kernel gave up a bounded wait (code %u): a look-back chain did not advance; results of the affected call are invalid", code);
}

static void free_retired_scratch() {
	State& s = state();
	for (size_t i = 0; i < s.retired_scratch_count; i++) hipFree(s.retired_scratch[i]);
	s.retired_scratch_count = 0;
}

// ---- roctx ranges, bound lazily so that the library loads where no profiler runtime exists ----
typedef int (*roctx_push_fn)(const char*);
typedef int (*roctx_pop_fn)(void);
static roctx_push_fn g_roctx_push = nullptr;
static roctx_pop_fn g_roctx_pop = nullptr;
static std::once_flag g_roctx_once;

static void bind_roctx() {
	const char* names[] = {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"};
	for (const char* n : names) {
		void* h = dlopen(n, RTLD_NOW | RTLD_GLOBAL);
		if (!h) continue;
		g_roctx_push = (roctx_push_fn)dlsym(h, "roctxRangePushA");
		g_roctx_pop = (roctx_pop_fn)dlsym(h, "roctxRangePop");
		if (g_roctx_push && g_roctx_pop) return;
		g_roctx_push = nullptr;
		g_roctx_pop = nullptr;
	}
}

// ---- code-object cache ----------------------------------------------------------------------
static uint64_t fnv1a(const void* data, size_t n, uint64_t h = 1469598103934665603ull) {
	const unsigned char* p = (const unsigned char*)data;
	for (size_t i = 0; i < n; i++) {
		h ^= p[i];
		h *= 1099511628211ull;
	}
	return h;
}

// TFHIP_CACHE_DIR, else a directory of this user's own under /tmp (one that another user created could not be written).
static std::string cache_dir() {
	const char* env = getenv("TFHIP_CACHE_DIR");
	std::string dir = env && *env ? env : "/tmp/tfhip_cache_" + std::to_string((long)getuid());
	mkdir(dir.c_str(), 0700);
	return dir;
}

// Code objects this process has compiled or read, by the same hash as the files: a program compiled twice in one
// process costs one compilation even where the directory cannot be written.
static std::mutex g_code_mutex;
static std::unordered_map<uint64_t, std::shared_ptr<std::vector<char>>> g_code_objects;
static std::vector<uint64_t> g_code_order;       // oldest first
constexpr size_t kMaxCodeObjectsKept = 1024;     // beyond that the oldest go (they are still in the directory)

static void keep_code_object(uint64_t h, const std::vector<char>& code) {  // g_code_mutex held
	if (!g_code_objects.count(h)) g_code_order.push_back(h);
	g_code_objects[h] = std::make_shared<std::vector<char>>(code);
	while (g_code_order.size() > kMaxCodeObjectsKept) {
		g_code_objects.erase(g_code_order.front());
		g_code_order.erase(g_code_order.begin());
	}
}

static bool read_file(const std::string& path, std::vector<char>& out) {
	FILE* f = fopen(path.c_str(), "rb");
	if (!f) return false;
	fseek(f, 0, SEEK_END);
	long n = ftell(f);
	fseek(f, 0, SEEK_SET);
	out.resize(n > 0 ? (size_t)n : 0);
	bool ok = n > 0 && fread(out.data(), 1, (size_t)n, f) == (size_t)n;
	fclose(f);
	return ok;
}

static void write_file_atomic(const std::string& path, const std::vector<char>& data) {
	std::string tmp = path + "." + std::to_string((long)getpid()) + ".tmp";
	FILE* f = fopen(tmp.c_str(), "wb");
	if (!f) return;
	bool ok = fwrite(data.data(), 1, data.size(), f) == data.size();
	fclose(f);
	if (ok)
		rename(tmp.c_str(), path.c_str());
	else
		unlink(tmp.c_str());
}

// Compiles `source` to a gfx950 code object (no device needed). Returns TFHIP_OK and fills `code`.
static int compile_to_code_object(const char* source, const char* kernel_name, const char* options, std::vector<char>& code) {
	std::vector<std::string> opts = {
	    "--offload-arch=gfx950", "-O3", "-std=c++17",
	    // Packed fp32 VALU forms are kept out of every kernel this library builds.
	    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
	};
	if (options) {
		std::string s(options);
		size_t i = 0;
		while (i < s.size()) {
			while (i < s.size() && s[i] == ' ') i++;
			size_t j = i;
			while (j < s.size() && s[j] != ' ') j++;
			if (j > i) opts.push_back(s.substr(i, j - i));
			i = j;
		}
	}
	std::vector<const char*> copts;
	for (auto& o : opts) copts.push_back(o.c_str());

	hiprtcProgram prog;
	std::string file = std::string(kernel_name) + ".hip";
	hiprtcResult r = hiprtcCreateProgram(&prog, source, file.c_str(), 0, nullptr, nullptr);
	if (r != HIPRTC_SUCCESS) return fail(TFHIP_ERR_COMPILE, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
	r = hiprtcCompileProgram(prog, (int)copts.size(), copts.data());
	if (r != HIPRTC_SUCCESS) {
		size_t log_size = 0;
		hiprtcGetProgramLogSize(prog, &log_size);
		std::string log(log_size, '\0');
		if (log_size) hiprtcGetProgramLog(prog, log.data());
		hiprtcDestroyProgram(&prog);
		// Same shape of message as the reference's compile failures: what failed, then the compiler output
		// (Backends/CPU/KernelCompiler.cpp:83-88, Backends/OpenGL/KernelManager.h:79-83).
		return fail(TFHIP_ERR_COMPILE, "Error compiling kernel %s: %s\n%.1800s", kernel_name, hiprtcGetErrorString(r), log.c_str());
	}
	size_t code_size = 0;
	hiprtcGetCodeSize(prog, &code_size);
	code.resize(code_size);
	hiprtcGetCode(prog, code.data());
	hiprtcDestroyProgram(&prog);
	return TFHIP_OK;
}

static __global__ void fill_u32_kernel(uint32_t* __restrict__ dst, uint32_t value, size_t n) {
	size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
	size_t stride = (size_t)gridDim.x * blockDim.x;
	for (; i < n; i += stride) dst[i] = value;
}

}  // namespace tfhip

using namespace tfhip;

// Argument blocks of module launches recorded since tfhip_graph_begin.
static std::vector<std::unique_ptr<unsigned char[]>> g_recorded_arguments;

extern "C" {

const char* tfhip_last_error(void) { return g_last_error.c_str(); }

int tfhip_init(int device) {
	State& s = state();
	if (s.initialized) {
		if (s.device == device) return TFHIP_OK;
		return fail(TFHIP_ERR_STATE, "already initialised on device %d; call tfhip_shutdown first", s.device);
	}
	int count = 0;
	TFHIP_CHECK(hipGetDeviceCount(&count));
	if (device < 0 || device >= count) return fail(TFHIP_ERR_ARG, "device %d out of range (%d visible)", device, count);
	TFHIP_CHECK(hipSetDevice(device));
	hipDeviceProp_t prop;
	TFHIP_CHECK(hipGetDeviceProperties(&prop, device));
	if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
		return fail(TFHIP_ERR_STATE, "device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
	{
		int rc = locate_static_scratch(device);
		if (rc) return rc;
	}
	TFHIP_CHECK(hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking));
	void* host_word = nullptr;
	TFHIP_CHECK(hipHostMalloc(&host_word, sizeof(uint32_t), hipHostMallocMapped));
	*(volatile uint32_t*)host_word = 0;
	void* dev_word = nullptr;
	TFHIP_CHECK(hipHostGetDevicePointer(&dev_word, host_word, 0));
	s.async_error_host = (volatile uint32_t*)host_word;
	s.async_error_dev = (uint32_t*)dev_word;
	s.device = device;
	s.compute_units = prop.multiProcessorCount;
	s.initialized = true;
	return TFHIP_OK;
}

static void stop_copy_pool();

int tfhip_shutdown(void) {
	State& s = state();
	if (!s.initialized) return TFHIP_OK;
	stop_copy_pool();
	hipStreamSynchronize(s.stream);
	if (s.scratch) hipFree(s.scratch);
	s.scratch = nullptr;
	s.scratch_bytes = 0;
	free_retired_scratch();
	s.live_graphs = 0;
	hipStreamDestroy(s.stream);
	s.stream = nullptr;
	for (int i = 0; i < 2; i++) {
		if (s.staging[i]) hipHostFree(s.staging[i]);
		if (s.staging_done[i]) hipEventDestroy(s.staging_done[i]);
		s.staging[i] = nullptr;
		s.staging_done[i] = nullptr;
	}
	if (s.async_error_host) hipHostFree((void*)s.async_error_host);
	s.async_error_host = nullptr;
	s.async_error_dev = nullptr;
	s.initialized = false;
	return TFHIP_OK;
}

int tfhip_device_info(char* name, size_t cap, int* compute_units, size_t* hbm_bytes) {
	TFHIP_REQUIRE_INIT();
	hipDeviceProp_t prop;
	TFHIP_CHECK(hipGetDeviceProperties(&prop, state().device));
	if (name && cap) {
		// some driver stacks report an empty marketing name: the architecture string still identifies the part
		if (prop.name[0])
			snprintf(name, cap, "%s (%s)", prop.name, prop.gcnArchName);
		else
			snprintf(name, cap, "%s, %d compute units", prop.gcnArchName, prop.multiProcessorCount);
	}
	if (compute_units) *compute_units = prop.multiProcessorCount;
	if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
	return TFHIP_OK;
}

int tfhip_malloc(void** dev_ptr, size_t n_words) {
	TFHIP_REQUIRE_INIT();
	if (!dev_ptr) return fail(TFHIP_ERR_ARG, "dev_ptr is null");
	if (n_words == 0) return fail(TFHIP_ERR_ARG, "Trying to allocate a tensor with size 0");
	*dev_ptr = nullptr;
	hipError_t e = hipMalloc(dev_ptr, n_words * sizeof(uint32_t));
	if (e != hipSuccess) {
		(void)hipGetLastError();
		return fail(TFHIP_ERR_HIP, "hipMalloc of %zu words failed: %s", n_words, hipGetErrorName(e));
	}
	return TFHIP_OK;
}

int tfhip_free(void* dev_ptr) {
	TFHIP_REQUIRE_INIT();
	if (!dev_ptr) return TFHIP_OK;
	TFHIP_REFUSE_WHILE_RECORDING("freeing device memory");
	// Work that still reads the buffer may be queued on the stream.
	TFHIP_CHECK(hipStreamSynchronize(state().stream));
	TFHIP_CHECK(hipFree(dev_ptr));
	return check_async_error();
}

// Large copies between pageable host memory and the device go through two pinned staging buffers: while the
// DMA engine moves one chunk, the host copies the next one into (or the previous one out of) the other buffer.
// The upload / readback of whole tensors is the reference's Python-side bottleneck as well
// (per-element std::function copies, Frontend/Python/PyTensorMemory.cpp:19-84).
constexpr size_t kStagingBytes = 8u << 20;
constexpr size_t kStagedCopyMin = 1u << 20;

// The host side of a staged copy (pageable memory <-> pinned buffer) is a memcpy; one thread moves 10-13 GB/s, less than
// the DMA engine does over the bus, so chunks are cut into slices that helper threads copy beside the caller. Reading
// back 1 GiB into memory the process has never touched (a fresh numpy array: every page is faulted in and zeroed on
// the way) runs at 34 GB/s with three helpers, 42 with seven, 45 with eleven; into touched memory, and uploading, at
// the bus's 51 GB/s with three already. Seven by default (fewer on a machine with fewer cores), TFHIP_COPY_HELPERS
// = 1..15 overrides.
class CopyPool {
 public:
	static constexpr int kMaxHelpers = 15;
	const int helpers_ = [] {
		const char* env = getenv("TFHIP_COPY_HELPERS");
		const int cores = (int)std::thread::hardware_concurrency();
		const int want = env ? atoi(env) : std::min(7, cores > 1 ? cores - 1 : 1);
		return std::max(1, std::min(kMaxHelpers, want));
	}();
	static CopyPool& get() {
		static CopyPool pool;
		return pool;
	}
	void copy(char* dst, const char* src, size_t bytes) {
		if (bytes < (1u << 20)) {
			memcpy(dst, src, bytes);
			return;
		}
		std::lock_guard<std::mutex> one_copy_at_a_time(call_mutex_);
		start();
		const size_t parts = (size_t)helpers_ + 1;
		const size_t slice = ((bytes + parts - 1) / parts + 4095) & ~(size_t)4095;  // parts * slice >= bytes
		{
			std::lock_guard<std::mutex> lock(mutex_);
			for (int i = 0; i < helpers_; i++) {
				const size_t at = std::min(bytes, slice * (size_t)(i + 1));
				const size_t end = std::min(bytes, slice * (size_t)(i + 2));
				slices_[i] = {dst + at, src + at, end - at};
			}
			pending_ = helpers_;
			generation_++;
		}
		work_.notify_all();
		memcpy(dst, src, std::min(bytes, slice));
		std::unique_lock<std::mutex> lock(mutex_);
		done_.wait(lock, [&] { return pending_ == 0; });
	}
	void stop() {
		std::lock_guard<std::mutex> no_copy_running(call_mutex_);
		{
			std::lock_guard<std::mutex> lock(mutex_);
			if (workers_.empty()) return;
			quit_ = true;
		}
		work_.notify_all();
		for (std::thread& t : workers_) t.join();
		workers_.clear();
		quit_ = false;
	}
	~CopyPool() { stop(); }

 private:
	struct Slice {
		char* dst;
		const char* src;
		size_t bytes;
	};
	void start() {
		if (!workers_.empty()) return;
		// A helper answers the requests made after it was started: it begins at the current generation, not at zero
		// (the pool is stopped by tfhip_shutdown and started again by the next large copy).
		uint64_t born;
		{
			std::lock_guard<std::mutex> lock(mutex_);
			born = generation_;
		}
		for (int i = 0; i < helpers_; i++) workers_.emplace_back([this, i, born] { run(i, born); });
	}
	void run(int id, uint64_t seen) {
		std::unique_lock<std::mutex> lock(mutex_);
		while (true) {
			work_.wait(lock, [&] { return quit_ || generation_ != seen; });
			if (quit_) return;
			seen = generation_;
			const Slice slice = slices_[id];
			lock.unlock();
			if (slice.bytes) memcpy(slice.dst, slice.src, slice.bytes);
			lock.lock();
			if (--pending_ == 0) done_.notify_one();
		}
	}
	std::vector<std::thread> workers_;
	std::mutex mutex_, call_mutex_;
	std::condition_variable work_, done_;
	Slice slices_[kMaxHelpers] = {};
	uint64_t generation_ = 0;
	int pending_ = 0;
	bool quit_ = false;
};

static void stop_copy_pool() { CopyPool::get().stop(); }

static int ensure_staging() {
	State& s = state();
	if (s.staging[0]) return TFHIP_OK;
	for (int i = 0; i < 2; i++) {
		TFHIP_CHECK(hipHostMalloc(&s.staging[i], kStagingBytes, hipHostMallocDefault));
		TFHIP_CHECK(hipEventCreateWithFlags(&s.staging_done[i], hipEventDisableTiming));
	}
	return TFHIP_OK;
}

int tfhip_h2d(void* dev_dst, size_t dst_offset_words, const uint32_t* host_src, size_t n_words) {
	TFHIP_REQUIRE_INIT();
	if (n_words == 0) return TFHIP_OK;
	if (!dev_dst || !host_src) return fail(TFHIP_ERR_ARG, "null pointer in tfhip_h2d");
	TFHIP_REFUSE_WHILE_RECORDING("a copy from host memory");
	State& s = state();
	char* dst = (char*)((uint32_t*)dev_dst + dst_offset_words);
	const char* src = (const char*)host_src;
	const size_t bytes = n_words * sizeof(uint32_t);
	if (bytes < kStagedCopyMin) {
		// Pageable source: the copy is staged by the runtime before the call returns, so the caller may reuse host_src.
		TFHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s.stream));
		TFHIP_CHECK(hipStreamSynchronize(s.stream));
		return check_async_error();
	}
	int rc = ensure_staging();
	if (rc) return rc;
	size_t done = 0;
	for (int i = 0; done < bytes; i++) {
		const int b = i & 1;
		const size_t chunk = bytes - done < kStagingBytes ? bytes - done : kStagingBytes;
		if (i >= 2) TFHIP_CHECK(hipEventSynchronize(s.staging_done[b]));  // the DMA that last read this buffer
		CopyPool::get().copy((char*)s.staging[b], src + done, chunk);
		TFHIP_CHECK(hipMemcpyAsync(dst + done, s.staging[b], chunk, hipMemcpyHostToDevice, s.stream));
		TFHIP_CHECK(hipEventRecord(s.staging_done[b], s.stream));
		done += chunk;
	}
	TFHIP_CHECK(hipStreamSynchronize(s.stream));
	return check_async_error();
}

int tfhip_d2h(uint32_t* host_dst, const void* dev_src, size_t src_offset_words, size_t n_words) {
	TFHIP_REQUIRE_INIT();
	if (n_words == 0) return TFHIP_OK;
	if (!dev_src || !host_dst) return fail(TFHIP_ERR_ARG, "null pointer in tfhip_d2h");
	TFHIP_REFUSE_WHILE_RECORDING("a copy to host memory");
	State& s = state();
	const char* src = (const char*)((const uint32_t*)dev_src + src_offset_words);
	char* dst = (char*)host_dst;
	const size_t bytes = n_words * sizeof(uint32_t);
	if (bytes < kStagedCopyMin) {
		TFHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s.stream));
		TFHIP_CHECK(hipStreamSynchronize(s.stream));
		return check_async_error();
	}
	int rc = ensure_staging();
	if (rc) return rc;
	// chunk i is in flight to staging[i & 1] while chunk i - 1 is copied out of the other buffer
	size_t issued = 0, drained = 0;
	size_t chunk_bytes[2] = {0, 0};
	for (int i = 0; drained < bytes; i++) {
		const int b = i & 1;
		if (issued < bytes) {
			const size_t chunk = bytes - issued < kStagingBytes ? bytes - issued : kStagingBytes;
			TFHIP_CHECK(hipMemcpyAsync(s.staging[b], src + issued, chunk, hipMemcpyDeviceToHost, s.stream));
			TFHIP_CHECK(hipEventRecord(s.staging_done[b], s.stream));
			chunk_bytes[b] = chunk;
			issued += chunk;
		}
		if (i >= 1) {
			const int p = b ^ 1;
			TFHIP_CHECK(hipEventSynchronize(s.staging_done[p]));
			CopyPool::get().copy(dst + drained, (const char*)s.staging[p], chunk_bytes[p]);
			drained += chunk_bytes[p];
		}
	}
	return check_async_error();
}

int tfhip_d2d(void* dev_dst, const void* dev_src, size_t n_words) {
	TFHIP_REQUIRE_INIT();
	if (n_words == 0) return TFHIP_OK;
	if (!dev_dst || !dev_src) return fail(TFHIP_ERR_ARG, "null pointer in tfhip_d2d");
	TFHIP_CHECK(hipMemcpyAsync(dev_dst, dev_src, n_words * sizeof(uint32_t), hipMemcpyDeviceToDevice, state().stream));
	return TFHIP_OK;
}

int tfhip_fill_u32(void* dev_dst, uint32_t value, size_t n_words) {
	TFHIP_REQUIRE_INIT();
	if (n_words == 0) return TFHIP_OK;
	if (!dev_dst) return fail(TFHIP_ERR_ARG, "null pointer in tfhip_fill_u32");
	size_t blocks = (n_words + 255) / 256;
	if (blocks > 65536) blocks = 65536;
	hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, state().stream, (uint32_t*)dev_dst, value, n_words);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

int tfhip_module_compile(const char* source, const char* kernel_name, const char* options, tfhip_kernel_t* out) {
	if (!source || !kernel_name || !out) return fail(TFHIP_ERR_ARG, "null argument in tfhip_module_compile");
	*out = nullptr;

	int rtc_major = 0, rtc_minor = 0;
	hiprtcVersion(&rtc_major, &rtc_minor);
	uint64_t h = fnv1a(source, strlen(source));
	h = fnv1a(kernel_name, strlen(kernel_name), h);
	if (options) h = fnv1a(options, strlen(options), h);
	h = fnv1a(&rtc_major, sizeof(int), h);
	h = fnv1a(&rtc_minor, sizeof(int), h);
	char hex[32];
	snprintf(hex, sizeof(hex), "%016llx", (unsigned long long)h);
	std::string path = cache_dir() + "/" + hex + ".hsaco";

	std::vector<char> code;
	const char* no_cache = getenv("TFHIP_NO_CACHE");
	const bool use_cache = !(no_cache && *no_cache == '1');
	bool from_cache = false;
	if (use_cache) {
		std::lock_guard<std::mutex> lock(g_code_mutex);
		auto it = g_code_objects.find(h);
		if (it != g_code_objects.end()) {
			code = *it->second;
			from_cache = true;
		}
	}
	if (from_cache) {
		if (access(path.c_str(), F_OK) != 0) write_file_atomic(path, code);  // e.g. another cache directory than before
	} else if (use_cache) {
		from_cache = read_file(path, code);
	}
	if (!from_cache) {
		int rc = compile_to_code_object(source, kernel_name, options, code);
		if (rc != TFHIP_OK) return rc;
		write_file_atomic(path, code);
	}
	if (use_cache) {
		std::lock_guard<std::mutex> lock(g_code_mutex);
		if (!g_code_objects.count(h)) keep_code_object(h, code);
	}

	// A handle without a loaded module is still useful on a machine with no GPU: it proves the source
	// compiles for gfx950. Launching it fails with TFHIP_ERR_STATE.
	tfhip_kernel* k = new tfhip_kernel();
	k->name = kernel_name;
	if (state().initialized) {
		hipError_t e = hipModuleLoadData(&k->module, code.data());
		if (e != hipSuccess && from_cache) {
			// Stale or truncated cache entry: rebuild once.
			(void)hipGetLastError();
			int rc = compile_to_code_object(source, kernel_name, options, code);
			if (rc != TFHIP_OK) {
				delete k;
				return rc;
			}
			write_file_atomic(path, code);
			{
				std::lock_guard<std::mutex> lock(g_code_mutex);
				keep_code_object(h, code);
			}
			e = hipModuleLoadData(&k->module, code.data());
		}
		if (e != hipSuccess) {
			delete k;
			return fail_hip(e, "hipModuleLoadData");
		}
		e = hipModuleGetFunction(&k->function, k->module, kernel_name);
		if (e != hipSuccess) {
			hipModuleUnload(k->module);
			delete k;
			return fail(TFHIP_ERR_COMPILE, "kernel symbol %s not found in compiled module (%s)", kernel_name, hipGetErrorName(e));
		}
	}
	*out = k;
	return TFHIP_OK;
}

int tfhip_module_get_kernel(tfhip_kernel_t kernel, const char* kernel_name, tfhip_kernel_t* out) {
	if (!kernel || !kernel_name || !out) return fail(TFHIP_ERR_ARG, "null argument in tfhip_module_get_kernel");
	*out = nullptr;
	tfhip_kernel* k = new tfhip_kernel();
	k->name = kernel_name;
	k->owns_module = false;
	k->module = kernel->module;
	if (kernel->module) {
		hipError_t e = hipModuleGetFunction(&k->function, kernel->module, kernel_name);
		if (e != hipSuccess) {
			delete k;
			return fail(TFHIP_ERR_COMPILE, "kernel symbol %s not found in compiled module (%s)", kernel_name, hipGetErrorName(e));
		}
	}
	*out = k;
	return TFHIP_OK;
}

int tfhip_module_unload(tfhip_kernel_t kernel) {
	if (!kernel) return TFHIP_OK;
	if (kernel->module && kernel->owns_module) {
		TFHIP_REFUSE_WHILE_RECORDING("unloading a module");
		hipStreamSynchronize(state().stream);
		hipModuleUnload(kernel->module);
	}
	delete kernel;
	return TFHIP_OK;
}

int tfhip_launch(tfhip_kernel_t kernel, uint32_t grid_x, uint32_t block_x, uint32_t block_y, uint32_t block_z,
                 void* const* buffers, size_t n_buffers, const uint32_t* vars, size_t n_vars) {
	TFHIP_REQUIRE_INIT();
	if (!kernel || !kernel->function) return fail(TFHIP_ERR_STATE, "kernel handle has no loaded function");
	if (grid_x == 0) return TFHIP_OK;  // nothing to do, as a zero-trip loop over groups on the CPU
	uint64_t threads = (uint64_t)block_x * block_y * block_z;
	if (threads == 0 || threads > 1024) return fail(TFHIP_ERR_ARG, "group size %ux%ux%u is outside 1..1024 threads", block_x, block_y, block_z);
	if (n_buffers > 64 || n_vars > 256) return fail(TFHIP_ERR_ARG, "too many kernel arguments (%zu buffers, %zu variables)", n_buffers, n_vars);
	if ((n_buffers && !buffers) || (n_vars && !vars)) return fail(TFHIP_ERR_ARG, "null argument array in tfhip_launch");

	// Kernel-argument segment: n_buffers 8-byte pointers, then the variable struct (4-byte aligned words).
	// While a graph is being recorded the block lives on the heap and is handed to the graph when recording ends.
	alignas(8) unsigned char stack_args[64 * 8 + 256 * 4];
	unsigned char* args = stack_args;
	if (state().capturing) {
		g_recorded_arguments.emplace_back(new unsigned char[sizeof(stack_args) + sizeof(size_t) + 5 * sizeof(void*)]);
		args = g_recorded_arguments.back().get();
	}
	size_t bytes = 0;
	for (size_t i = 0; i < n_buffers; i++) {
		if (!buffers[i]) return fail(TFHIP_ERR_ARG, "buffer %zu of kernel %s is null", i, kernel->name.c_str());
		memcpy(args + bytes, &buffers[i], 8);
		bytes += 8;
	}
	if (n_vars) {
		memcpy(args + bytes, vars, n_vars * 4);
		bytes += n_vars * 4;
	}
	size_t* bytes_ptr = &bytes;
	void* stack_config[5];
	void** config = stack_config;
	if (state().capturing) {
		// the size word and the five-entry launch configuration live behind the arguments in the same heap block, so
		// that nothing a recorded launch was given points into this call's stack frame
		bytes_ptr = reinterpret_cast<size_t*>(args + sizeof(stack_args));
		*bytes_ptr = bytes;
		config = reinterpret_cast<void**>(args + sizeof(stack_args) + sizeof(size_t));
	}
	config[0] = HIP_LAUNCH_PARAM_BUFFER_POINTER;
	config[1] = args;
	config[2] = HIP_LAUNCH_PARAM_BUFFER_SIZE;
	config[3] = bytes_ptr;
	config[4] = HIP_LAUNCH_PARAM_END;
	TFHIP_CHECK(hipModuleLaunchKernel(kernel->function, grid_x, 1, 1, block_x, block_y, block_z, 0, state().stream, nullptr, config));
	return TFHIP_OK;
}

int tfhip_launch_batch(tfhip_kernel_t kernel, uint32_t grid_x, uint32_t calls, uint32_t block_x, const void* arguments, size_t bytes) {
	TFHIP_REQUIRE_INIT();
	if (!kernel || !kernel->function) return fail(TFHIP_ERR_STATE, "kernel handle has no loaded function");
	if (grid_x == 0 || calls == 0) return TFHIP_OK;
	if (block_x == 0 || block_x > 1024) return fail(TFHIP_ERR_ARG, "group size %u is outside 1..1024 threads", block_x);
	if (calls > 65535) return fail(TFHIP_ERR_ARG, "more than 65535 dispatches in one launch (%u)", calls);
	if (!arguments || bytes == 0 || bytes > 4096) return fail(TFHIP_ERR_ARG, "argument array of %zu bytes (1..4096 allowed)", bytes);
	// As in tfhip_launch: while a graph is being recorded the argument block lives on the heap and is handed to the graph.
	alignas(8) unsigned char stack_args[4096];
	unsigned char* args = stack_args;
	size_t size = bytes;
	size_t* size_ptr = &size;
	void* stack_config[5];
	void** config = stack_config;
	if (state().capturing) {
		g_recorded_arguments.emplace_back(new unsigned char[sizeof(stack_args) + sizeof(size_t) + 5 * sizeof(void*)]);
		args = g_recorded_arguments.back().get();
		size_ptr = reinterpret_cast<size_t*>(args + sizeof(stack_args));
		*size_ptr = bytes;
		config = reinterpret_cast<void**>(args + sizeof(stack_args) + sizeof(size_t));
	}
	memcpy(args, arguments, bytes);
	config[0] = HIP_LAUNCH_PARAM_BUFFER_POINTER;
	config[1] = args;
	config[2] = HIP_LAUNCH_PARAM_BUFFER_SIZE;
	config[3] = size_ptr;
	config[4] = HIP_LAUNCH_PARAM_END;
	TFHIP_CHECK(hipModuleLaunchKernel(kernel->function, grid_x, calls, 1, block_x, 1, 1, 0, state().stream, nullptr, config));
	return TFHIP_OK;
}

int tfhip_sync(void) {
	TFHIP_REQUIRE_INIT();
	TFHIP_REFUSE_WHILE_RECORDING("waiting for the stream");
	TFHIP_CHECK(hipStreamSynchronize(state().stream));
	return check_async_error();
}

// ---- recorded graphs ---------------------------------------------------------------------------------------

int tfhip_graph_begin(void) {
	TFHIP_REQUIRE_INIT();
	State& s = state();
	if (s.capturing) return fail(TFHIP_ERR_STATE, "a graph is already being recorded");
	g_recorded_arguments.clear();
	// Relaxed mode: allocations made by the host side while recording (a pool that has to grow) stay legal.
	TFHIP_CHECK(hipStreamBeginCapture(s.stream, hipStreamCaptureModeRelaxed));
	s.capturing = true;
	return TFHIP_OK;
}

int tfhip_graph_end(tfhip_graph_t* out) {
	TFHIP_REQUIRE_INIT();
	State& s = state();
	if (!s.capturing) return fail(TFHIP_ERR_STATE, "no graph is being recorded");
	s.capturing = false;
	hipGraph_t graph = nullptr;
	hipError_t e = hipStreamEndCapture(s.stream, &graph);
	if (e != hipSuccess) {
		g_recorded_arguments.clear();
		return fail_hip(e, "hipStreamEndCapture");
	}
	if (!out) {  // recording abandoned
		if (graph) hipGraphDestroy(graph);
		g_recorded_arguments.clear();
		return TFHIP_OK;
	}
	tfhip_graph* g = new tfhip_graph();
	g->graph = graph;
	g->arguments = std::move(g_recorded_arguments);
	g_recorded_arguments.clear();
	e = hipGraphInstantiate(&g->exec, graph, nullptr, nullptr, 0);
	if (e != hipSuccess) {
		hipGraphDestroy(graph);
		delete g;
		return fail_hip(e, "hipGraphInstantiate");
	}
	s.live_graphs++;
	*out = g;
	return TFHIP_OK;
}

int tfhip_graph_node_count(tfhip_graph_t graph, size_t* nodes) {
	if (!graph || !nodes) return fail(TFHIP_ERR_ARG, "null argument in tfhip_graph_node_count");
	TFHIP_CHECK(hipGraphGetNodes(graph->graph, nullptr, nodes));
	return TFHIP_OK;
}

int tfhip_graph_launch(tfhip_graph_t graph) {
	TFHIP_REQUIRE_INIT();
	if (!graph || !graph->exec) return fail(TFHIP_ERR_ARG, "graph handle is null");
	TFHIP_REFUSE_WHILE_RECORDING("launching a graph");
	TFHIP_CHECK(hipGraphLaunch(graph->exec, state().stream));
	return TFHIP_OK;
}

int tfhip_graph_destroy(tfhip_graph_t graph) {
	if (!graph) return TFHIP_OK;
	if (state().initialized) hipStreamSynchronize(state().stream);
	if (graph->exec) hipGraphExecDestroy(graph->exec);
	if (graph->graph) hipGraphDestroy(graph->graph);
	delete graph;
	State& s = state();
	if (s.live_graphs > 0 && --s.live_graphs == 0) free_retired_scratch();  // the stream is idle: nothing reads them any more
	return TFHIP_OK;
}

int tfhip_scratch_info(size_t* bytes, size_t* retired_buffers, size_t* live_graphs) {
	State& s = state();
	if (bytes) *bytes = s.scratch_bytes;
	if (retired_buffers) *retired_buffers = s.retired_scratch_count;
	if (live_graphs) *live_graphs = s.live_graphs;
	return TFHIP_OK;
}

int tfhip_scratch_reserve(size_t bytes) {
	TFHIP_REQUIRE_INIT();
	return scratch(bytes) ? TFHIP_OK : TFHIP_ERR_HIP;
}

int tfhip_test_raise_async_error(uint32_t code) {
	TFHIP_REQUIRE_INIT();
	*state().async_error_host = code;
	return TFHIP_OK;
}

int tfhip_range_push(const char* name) {
	std::call_once(g_roctx_once, bind_roctx);
	if (g_roctx_push) g_roctx_push(name ? name : "");
	return TFHIP_OK;
}

int tfhip_range_pop(void) {
	std::call_once(g_roctx_once, bind_roctx);
	if (g_roctx_pop) g_roctx_pop();
	return TFHIP_OK;
}

int tfhip_event_create(tfhip_event_t* out) {
	TFHIP_REQUIRE_INIT();
	if (!out) return fail(TFHIP_ERR_ARG, "out is null");
	tfhip_event* e = new tfhip_event();
	hipError_t err = hipEventCreate(&e->ev);
	if (err != hipSuccess) {
		delete e;
		return fail_hip(err, "hipEventCreate");
	}
	*out = e;
	return TFHIP_OK;
}

int tfhip_event_destroy(tfhip_event_t ev) {
	if (!ev) return TFHIP_OK;
	hipEventDestroy(ev->ev);
	delete ev;
	return TFHIP_OK;
}

int tfhip_event_record(tfhip_event_t ev) {
	TFHIP_REQUIRE_INIT();
	if (!ev) return fail(TFHIP_ERR_ARG, "event is null");
	TFHIP_CHECK(hipEventRecord(ev->ev, state().stream));
	return TFHIP_OK;
}

int tfhip_event_elapsed_ms(tfhip_event_t start, tfhip_event_t stop, float* ms) {
	TFHIP_REQUIRE_INIT();
	if (!start || !stop || !ms) return fail(TFHIP_ERR_ARG, "null argument in tfhip_event_elapsed_ms");
	TFHIP_CHECK(hipEventSynchronize(stop->ev));
	TFHIP_CHECK(hipEventElapsedTime(ms, start->ev, stop->ev));
	return check_async_error();
}

}  // extern "C"
