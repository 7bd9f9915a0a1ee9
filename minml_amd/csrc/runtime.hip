/*
 * runtime.hip — device identity, context (one stream + growable device scratch), events and memory calls of the HIP backend.
 * Behavioural counterpart of reference src/backend/cuda/{cuda_properties.cpp, cuda_context.cpp, cuda_event.cpp, cuda_memory.cu}.
 */
#include "common.hpp"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <map>
#include <sstream>
#include <string>
#include <utility>
#include <vector>

namespace
{
	using namespace mlhip;

	const std::vector<hipDeviceProp_t>& device_properties()
	{
		static const std::vector<hipDeviceProp_t> props = []()
		{
			std::vector<hipDeviceProp_t> result;
			int count = 0;
			if (hipGetDeviceCount(&count) != hipSuccess)
			{
				(void) hipGetLastError(); /* "no device" is an answer, not an error state to leave behind */
				count = 0;
			}
			for (int i = 0; i < count; i++)
			{
				hipDeviceProp_t p;
				if (hipGetDeviceProperties(&p, i) == hipSuccess)
					result.push_back(p);
			}
			return result;
		}();
		return props;
	}
	const std::vector<std::string>& device_infos()
	{
		static const std::vector<std::string> infos = []()
		{
			std::vector<std::string> result;
			for (const hipDeviceProp_t &p : device_properties())
			{
				std::ostringstream os;
				os << p.name << " (" << p.gcnArchName << ") : " << p.multiProcessorCount << " x CU with " << (p.totalGlobalMem >> 20) << "MB of memory";
				result.push_back(os.str());
			}
			return result;
		}();
		return infos;
	}
	const std::vector<std::string>& device_features()
	{
		static const std::vector<std::string> features = []()
		{
			std::vector<std::string> result;
			for (const hipDeviceProp_t &p : device_properties())
			{
				std::ostringstream os;
				os << "name : " << p.name << '\n';
				os << "arch : " << p.gcnArchName << '\n';
				os << "compute units : " << p.multiProcessorCount << '\n';
				os << "wavefront size : " << p.warpSize << '\n';
				os << "LDS per workgroup : " << p.sharedMemPerBlock << '\n';
				os << "L2 cache : " << p.l2CacheSize << '\n';
				os << "memory clock [kHz] : " << p.memoryClockRate << '\n';
				os << "memory bus width : " << p.memoryBusWidth << '\n';
				os << "core clock [kHz] : " << p.clockRate << '\n';
				os << "global memory [MB] : " << (p.totalGlobalMem >> 20) << '\n';
				result.push_back(os.str());
			}
			return result;
		}();
		return features;
	}

	void use_device(int index)
	{
		MLHIP_CHECK(hipSetDevice(index));
	}

	template<typename T>
	__global__ void kernel_fill(T *dst, size_t elements, T value)
	{
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < elements; i += stride)
			dst[i] = value;
	}
	template<typename T>
	void launch_fill(hipStream_t stream, void *dst, size_t bytes, const void *pattern)
	{
		const size_t elements = bytes / sizeof(T);
		if (elements == 0)
			return;
		T v;
		std::memcpy(&v, pattern, sizeof(T));
		const size_t blocks = (elements + 255) / 256;
		const unsigned int grid = static_cast<unsigned int>(blocks < 65536 ? blocks : 65536);
		hipLaunchKernelGGL(kernel_fill<T>, dim3(grid), dim3(256), 0, stream, reinterpret_cast<T*>(dst), elements, v);
		MLHIP_CHECK(hipGetLastError());
	}
}

namespace mlhip
{
	int device_compute_units()
	{
		int device = 0;
		MLHIP_CHECK(hipGetDevice(&device));
		const std::vector<hipDeviceProp_t> &props = device_properties();
		if (device < 0 || device >= static_cast<int>(props.size()))
			fail_runtime("HIP backend: no current device");
		return props[device].multiProcessorCount;
	}
	void ensure_dynamic_lds(const void *kernel, int bytes)
	{
		/* largest size granted so far per (device, kernel): callers ask for shape-dependent sizes, so a later, larger request must raise
		 * the limit again; the limit never goes below the 64 KB every kernel has by default */
		static std::mutex guard;
		static std::map<std::pair<int, const void*>, int> granted;
		constexpr int DEFAULT_LIMIT = 64 * 1024;
		if (bytes <= DEFAULT_LIMIT)
			return;
		int device = 0;
		MLHIP_CHECK(hipGetDevice(&device));
		std::lock_guard<std::mutex> lock(guard);
		int &limit = granted[std::make_pair(device, kernel)];
		if (bytes > limit)
		{
			MLHIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
			limit = bytes;
		}
	}
	void* get_workspace(mlContext_t context, size_t bytes)
	{
		Context *ctx = get(context);
		if (ctx->workspace_size < bytes)
		{
			use_device(ctx->device_index);
			MLHIP_CHECK(hipStreamSynchronize(ctx->stream)); /* earlier kernels may still read the old block */
			if (ctx->workspace != nullptr)
				MLHIP_CHECK(hipFree(ctx->workspace));
			ctx->workspace = nullptr;
			ctx->workspace_size = 0;
			const size_t rounded = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
			MLHIP_CHECK(hipMalloc(&ctx->workspace, rounded));
			ctx->workspace_size = rounded;
		}
		return ctx->workspace;
	}
}

namespace mlhip
{
	namespace
	{
		std::atomic<int> error_capture { 0 };
		std::mutex error_mutex;
		/* 0 none, 1 std::logic_error, 2 std::runtime_error or another std::exception, 3 anything else; written under the mutex, read by
		 * hosts through hip_error_flag_address without it, hence atomic */
		std::atomic<int> error_kind { 0 };
		static_assert(sizeof(std::atomic<int>) == sizeof(int) && std::atomic<int>::is_always_lock_free, "the error flag is exposed as a plain int");
		std::string error_message;
	}
	int& nested_entry_depth()
	{
		thread_local int depth = 0;
		return depth;
	}
	bool capture_current_exception()
	{
		if (error_capture.load() == 0 || nested_entry_depth() > 0)
			return false;
		int kind = 3;
		std::string message = "unknown exception";
		try
		{
			throw;
		}
		catch (const std::logic_error &e)
		{
			kind = 1;
			message = e.what();
		}
		catch (const std::exception &e)
		{
			kind = 2;
			message = e.what();
		}
		catch (...)
		{
		}
		std::lock_guard<std::mutex> lock(error_mutex);
		if (error_kind.load() == 0)
		{ /* the first failure since the last hip_take_last_error is the one reported */
			error_message = message;
			error_kind.store(kind);
		}
		return true;
	}
}

extern "C"
{
	void hip_set_error_capture(int enabled)
	{
		mlhip::error_capture.store(enabled != 0 ? 1 : 0);
	}
	const int* hip_error_flag_address(void)
	{
		return reinterpret_cast<const int*>(&mlhip::error_kind);
	}
	int hip_take_last_error(char *buffer, int size)
	{
		std::lock_guard<std::mutex> lock(mlhip::error_mutex);
		const int kind = mlhip::error_kind.load();
		if (buffer != nullptr && size > 0)
		{
			const size_t n = std::min(static_cast<size_t>(size - 1), mlhip::error_message.size());
			std::memcpy(buffer, mlhip::error_message.data(), n);
			buffer[n] = 0;
		}
		mlhip::error_kind.store(0);
		mlhip::error_message.clear();
		return kind;
	}

	using namespace mlhip;

	int hip_get_number_of_devices(void)
	try
	{
		return static_cast<int>(device_properties().size());
	}
	catch (...)
	{
		return mlhip::entry_failed<int>();
	}
	int hip_get_memory(int index)
	try
	{
		if (index < 0 || index >= hip_get_number_of_devices())
			return 0;
		return static_cast<int>(device_properties()[index].totalGlobalMem >> 20);
	}
	catch (...)
	{
		return mlhip::entry_failed<int>();
	}
	bool hip_supports_type(int index, mlDataType_t dtype)
	try
	{
		if (index < 0 || index >= hip_get_number_of_devices())
			return false;
		switch (dtype)
		{
			case DTYPE_FLOAT16:
			case DTYPE_FLOAT32:
			case DTYPE_INT32:
			case DTYPE_INT8:
				return true;
			default:
				return false;
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<bool>();
	}
	const char* hip_get_device_info(int index)
	try
	{
		if (index < 0 || index >= hip_get_number_of_devices())
			return nullptr;
		return device_infos()[index].c_str();
	}
	catch (...)
	{
		return mlhip::entry_failed<const char*>();
	}
	const char* hip_get_device_features(int index)
	try
	{
		if (index < 0 || index >= hip_get_number_of_devices())
			return nullptr;
		return device_features()[index].c_str();
	}
	catch (...)
	{
		return mlhip::entry_failed<const char*>();
	}
	void hip_enable_tf32(mlContext_t context, bool b)
	try
	{
		(void) context;
		(void) b;
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	mlContext_t hip_create_context(int device_index)
	try
	{
		if (device_index < 0 || device_index >= hip_get_number_of_devices())
			fail_logic("HIP backend: hip_create_context: no such device");
		use_device(device_index);
		Context *ctx = new Context();
		ctx->device_index = device_index;
		/* a blocking stream, as in the reference (src/backend/cuda/utils.cpp:115): context-less (synchronous) copies order against it */
		MLHIP_CHECK(hipStreamCreate(&ctx->stream));
		/* set-up that entry points must not do on their first call (a caller may be recording a graph by then): the device address of the
		 * library's static device memory and the LDS limits of the kernels that use it */
		prepare_static_memory(device_index);
		return ctx;
	}
	catch (...)
	{
		return mlhip::entry_failed<mlContext_t>();
	}
	void hip_synchronize_with_context(mlContext_t context)
	try
	{
		MLHIP_CHECK(hipStreamSynchronize(stream_of(context)));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	bool hip_is_context_ready(mlContext_t context)
	try
	{
		const hipError_t status = hipStreamQuery(stream_of(context));
		if (status == hipSuccess)
			return true;
		if (status == hipErrorNotReady)
			return false;
		check(status, "hipStreamQuery");
		return false;
	}
	catch (...)
	{
		return mlhip::entry_failed<bool>();
	}
	void hip_destroy_context(mlContext_t context)
	try
	{
		if (context == nullptr)
			return;
		Context *ctx = get(context);
		use_device(ctx->device_index);
		MLHIP_CHECK(hipStreamSynchronize(ctx->stream));
		if (ctx->workspace != nullptr)
			MLHIP_CHECK(hipFree(ctx->workspace));
		MLHIP_CHECK(hipStreamDestroy(ctx->stream));
		delete ctx;
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void* hip_get_stream(mlContext_t context)
	try
	{
		return reinterpret_cast<void*>(stream_of(context));
	}
	catch (...)
	{
		return mlhip::entry_failed<void*>();
	}

	/*
	 * A sequence of calls on a context recorded once and replayed as one HIP graph: for passes that are a chain of many short dependent
	 * launches (small batches), where the host's launch cost per kernel is what bounds the pass. Every entry point of this library only
	 * launches kernels and copies on the context's stream, so a pass may be recorded as it is; what must not happen while recording is
	 * anything that synchronises or allocates (first-use work such as weight transforms and workspace growth: run one pass before).
	 */
	struct Graph
	{
			int device_index = 0;
			hipGraph_t graph = nullptr;
			hipGraphExec_t exec = nullptr;
	};
	void hip_graph_begin_capture(mlContext_t context)
	try
	{
		Context *ctx = get(context);
		use_device(ctx->device_index);
		MLHIP_CHECK(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	mlGraph_t hip_graph_end_capture(mlContext_t context)
	try
	{
		Context *ctx = get(context);
		Graph *g = new Graph();
		g->device_index = ctx->device_index;
		const hipError_t status = hipStreamEndCapture(ctx->stream, &g->graph);
		if (status != hipSuccess || g->graph == nullptr)
		{
			delete g;
			check(status == hipSuccess ? hipErrorUnknown : status, "hipStreamEndCapture");
		}
		const hipError_t inst = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
		if (inst != hipSuccess)
		{
			(void) hipGraphDestroy(g->graph);
			delete g;
			check(inst, "hipGraphInstantiate");
		}
		return g;
	}
	catch (...)
	{
		return mlhip::entry_failed<mlGraph_t>();
	}
	void hip_graph_launch(mlContext_t context, mlGraph_t graph)
	try
	{
		MLHIP_REQUIRE(graph != nullptr, "hip_graph_launch: null graph");
		Context *ctx = get(context);
		MLHIP_REQUIRE(reinterpret_cast<Graph*>(graph)->device_index == ctx->device_index,
				"hip_graph_launch: the graph was recorded on another device than the context's");
		use_device(ctx->device_index);
		MLHIP_CHECK(hipGraphLaunch(reinterpret_cast<Graph*>(graph)->exec, ctx->stream));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_graph_destroy(mlGraph_t graph)
	try
	{
		if (graph == nullptr)
			return;
		Graph *g = reinterpret_cast<Graph*>(graph);
		MLHIP_CHECK(hipGraphExecDestroy(g->exec));
		MLHIP_CHECK(hipGraphDestroy(g->graph));
		delete g;
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	mlEvent_t hip_create_event(mlContext_t context)
	try
	{
		Context *ctx = get(context);
		use_device(ctx->device_index);
		Event *ev = new Event();
		ev->device_index = ctx->device_index;
		MLHIP_CHECK(hipEventCreate(&ev->event));
		MLHIP_CHECK(hipEventRecord(ev->event, ctx->stream));
		return ev;
	}
	catch (...)
	{
		return mlhip::entry_failed<mlEvent_t>();
	}
	double hip_get_time_between_events(mlEvent_t start, mlEvent_t end)
	try
	{
		MLHIP_REQUIRE(start != nullptr && end != nullptr, "null event");
		float ms = 0.0f;
		MLHIP_CHECK(hipEventElapsedTime(&ms, reinterpret_cast<Event*>(start)->event, reinterpret_cast<Event*>(end)->event));
		return static_cast<double>(ms) * 1.0e-3;
	}
	catch (...)
	{
		return mlhip::entry_failed<double>();
	}
	void hip_wait_for_event(mlEvent_t event)
	try
	{
		MLHIP_REQUIRE(event != nullptr, "null event");
		MLHIP_CHECK(hipEventSynchronize(reinterpret_cast<Event*>(event)->event));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	bool hip_is_event_ready(mlEvent_t event)
	try
	{
		MLHIP_REQUIRE(event != nullptr, "null event");
		const hipError_t status = hipEventQuery(reinterpret_cast<Event*>(event)->event);
		if (status == hipSuccess)
			return true;
		if (status == hipErrorNotReady)
			return false;
		check(status, "hipEventQuery");
		return false;
	}
	catch (...)
	{
		return mlhip::entry_failed<bool>();
	}
	void hip_destroy_event(mlEvent_t event)
	try
	{
		if (event == nullptr)
			return;
		Event *ev = reinterpret_cast<Event*>(event);
		MLHIP_CHECK(hipEventDestroy(ev->event));
		delete ev;
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	void* hip_malloc(int device_index, size_t count)
	try
	{
		if (count == 0)
			return nullptr;
		use_device(device_index);
		void *result = nullptr;
		MLHIP_CHECK(hipMalloc(&result, count));
		return result;
	}
	catch (...)
	{
		return mlhip::entry_failed<void*>();
	}
	void hip_page_lock(void *ptr, size_t count)
	try
	{
		(void) ptr;
		(void) count;
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_page_unlock(void *ptr)
	try
	{
		(void) ptr;
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_free(void *ptr)
	try
	{
		if (ptr != nullptr)
			MLHIP_CHECK(hipFree(ptr));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void* hip_create_view(void *src, size_t offset, size_t count)
	try
	{
		(void) count;
		if (src == nullptr)
			return nullptr;
		return reinterpret_cast<uint8_t*>(src) + offset;
	}
	catch (...)
	{
		return mlhip::entry_failed<void*>();
	}
	void hip_destroy_view(void *ptr)
	try
	{
		(void) ptr;
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_memset(mlContext_t context, void *dst, size_t dst_offset, size_t dst_count, const void *src, size_t src_count)
	try
	{
		MLHIP_REQUIRE(dst != nullptr, "hip_memset: null destination");
		if (dst_count == 0)
			return;
		uint8_t *tmp_dst = reinterpret_cast<uint8_t*>(dst) + dst_offset;
		hipStream_t stream = (context == nullptr) ? nullptr : stream_of(context);

		static const uint64_t zero = 0;
		if (src == nullptr || src_count == 0)
		{
			src = &zero;
			src_count = 1;
			if (dst_count % 8 == 0 && reinterpret_cast<uintptr_t>(tmp_dst) % 8 == 0)
				src_count = 8;
			else if (dst_count % 4 == 0 && reinterpret_cast<uintptr_t>(tmp_dst) % 4 == 0)
				src_count = 4;
		}
		MLHIP_REQUIRE(dst_count % src_count == 0, "hip_memset: destination size is not a multiple of the pattern size");
		MLHIP_REQUIRE(reinterpret_cast<uintptr_t>(tmp_dst) % src_count == 0, "hip_memset: destination is not aligned to the pattern size");
		switch (src_count)
		{
			case 1:
				launch_fill<uint8_t>(stream, tmp_dst, dst_count, src);
				break;
			case 2:
				launch_fill<uint16_t>(stream, tmp_dst, dst_count, src);
				break;
			case 4:
				launch_fill<uint32_t>(stream, tmp_dst, dst_count, src);
				break;
			case 8:
				launch_fill<uint64_t>(stream, tmp_dst, dst_count, src);
				break;
			default:
				fail_logic("HIP backend: hip_memset: pattern must be 1, 2, 4 or 8 bytes");
		}
		if (context == nullptr)
			MLHIP_CHECK(hipDeviceSynchronize());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_memcpy_within_device(mlContext_t context, void *dst, size_t dst_offset, const void *src, size_t src_offset, size_t count)
	try
	{
		if (count == 0)
			return;
		MLHIP_REQUIRE(dst != nullptr && src != nullptr, "hip_memcpy_within_device: null pointer");
		uint8_t *d = reinterpret_cast<uint8_t*>(dst) + dst_offset;
		const uint8_t *s = reinterpret_cast<const uint8_t*>(src) + src_offset;
		if (context == nullptr)
			MLHIP_CHECK(hipMemcpy(d, s, count, hipMemcpyDeviceToDevice));
		else
			MLHIP_CHECK(hipMemcpyAsync(d, s, count, hipMemcpyDeviceToDevice, stream_of(context)));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_memcpy_from_host(mlContext_t context, void *dst, size_t dst_offset, const void *src, size_t count)
	try
	{
		if (count == 0)
			return;
		MLHIP_REQUIRE(dst != nullptr && src != nullptr, "hip_memcpy_from_host: null pointer");
		uint8_t *d = reinterpret_cast<uint8_t*>(dst) + dst_offset;
		if (context == nullptr)
			MLHIP_CHECK(hipMemcpy(d, src, count, hipMemcpyHostToDevice));
		else
			MLHIP_CHECK(hipMemcpyAsync(d, src, count, hipMemcpyHostToDevice, stream_of(context)));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_memcpy_to_host(mlContext_t context, void *dst, const void *src, size_t src_offset, size_t count)
	try
	{
		if (count == 0)
			return;
		MLHIP_REQUIRE(dst != nullptr && src != nullptr, "hip_memcpy_to_host: null pointer");
		const uint8_t *s = reinterpret_cast<const uint8_t*>(src) + src_offset;
		if (context == nullptr)
			MLHIP_CHECK(hipMemcpy(dst, s, count, hipMemcpyDeviceToHost));
		else
			MLHIP_CHECK(hipMemcpyAsync(dst, s, count, hipMemcpyDeviceToHost, stream_of(context)));
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(get_number_of_devices)
MLHIP_ALSO_AS_CUDA(get_memory)
MLHIP_ALSO_AS_CUDA(supports_type)
MLHIP_ALSO_AS_CUDA(get_device_info)
MLHIP_ALSO_AS_CUDA(get_device_features)
MLHIP_ALSO_AS_CUDA(enable_tf32)
MLHIP_ALSO_AS_CUDA(create_context)
MLHIP_ALSO_AS_CUDA(synchronize_with_context)
MLHIP_ALSO_AS_CUDA(is_context_ready)
MLHIP_ALSO_AS_CUDA(destroy_context)
MLHIP_ALSO_AS_CUDA(create_event)
MLHIP_ALSO_AS_CUDA(get_time_between_events)
MLHIP_ALSO_AS_CUDA(wait_for_event)
MLHIP_ALSO_AS_CUDA(is_event_ready)
MLHIP_ALSO_AS_CUDA(destroy_event)
MLHIP_ALSO_AS_CUDA(malloc)
MLHIP_ALSO_AS_CUDA(page_lock)
MLHIP_ALSO_AS_CUDA(page_unlock)
MLHIP_ALSO_AS_CUDA(free)
MLHIP_ALSO_AS_CUDA(create_view)
MLHIP_ALSO_AS_CUDA(destroy_view)
MLHIP_ALSO_AS_CUDA(memset)
MLHIP_ALSO_AS_CUDA(memcpy_within_device)
MLHIP_ALSO_AS_CUDA(memcpy_from_host)
MLHIP_ALSO_AS_CUDA(memcpy_to_host)
