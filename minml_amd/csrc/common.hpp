/*
 * common.hpp — shared host-side plumbing of the HIP backend: the context object behind mlContext_t, descriptor helpers
 * and status checking. Counterpart of reference src/backend/cuda/utils.hpp:28-66 (Context{stream, workspace}) and
 * include/minml/backend/backend_utils.hpp (size_of, volume, is_transpose).
 */
#ifndef MINML_AMD_COMMON_HPP_
#define MINML_AMD_COMMON_HPP_

#include "../../include/minml_hip_backend.h"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstddef>
#include <stdexcept>
#include <string>
#include <type_traits>

namespace mlhip
{
	struct Context
	{
			int device_index = 0;
			hipStream_t stream = nullptr;
			void *workspace = nullptr; /* lazily allocated device scratch owned by the context */
			size_t workspace_size = 0;
	};

	struct Event
	{
			int device_index = 0;
			hipEvent_t event = nullptr;
	};

	/*
	 * Errors leave every entry point as C++ exceptions, as in the reference. A host that cannot catch them (ctypes and other C FFIs: the
	 * exception would end the process) switches capture on with hip_set_error_capture(1): the entry point then records the exception,
	 * returns normally (a zero / null value where it returns one), and the host asks hip_take_last_error afterwards. Every entry point
	 * is a function-try-block whose handler calls entry_failed; with capture off the handler rethrows and nothing changes.
	 */
	bool capture_current_exception(); /* runtime.hip; call from a catch handler only */
	/*
	 * Some entry points are written in terms of others (gemm_v2 -> gemm, winograd_layer_forward -> gemm_batched + fused transform ...).
	 * Such a function holds a NestedEntryCalls object while it calls them: as long as one exists on the calling thread, an inner entry
	 * point never captures — its handler rethrows, the exception unwinds to the outermost function-try-block (whose handler runs after
	 * the object is gone) and is captured there, so a failed outer call has launched nothing after the failure.
	 */
	int& nested_entry_depth(); /* runtime.hip; thread-local */
	struct NestedEntryCalls
	{
			NestedEntryCalls()
			{
				++nested_entry_depth();
			}
			~NestedEntryCalls()
			{
				--nested_entry_depth();
			}
			NestedEntryCalls(const NestedEntryCalls&) = delete;
			NestedEntryCalls& operator=(const NestedEntryCalls&) = delete;
	};
	template<typename R>
	inline R entry_failed()
	{
		if (!capture_current_exception())
			throw;
		if constexpr (!std::is_void<R>::value)
			return R();
	}

	[[noreturn]] inline void fail_runtime(const std::string &msg)
	{
		throw std::runtime_error(msg);
	}
	[[noreturn]] inline void fail_logic(const std::string &msg)
	{
		throw std::logic_error(msg);
	}

	inline void check(hipError_t status, const char *what)
	{
		if (status != hipSuccess)
			fail_runtime(std::string("HIP backend: ") + what + " failed: " + hipGetErrorString(status));
	}
#define MLHIP_CHECK(expr) ::mlhip::check((expr), #expr)
#define MLHIP_REQUIRE(cond, msg) do { if (!(cond)) ::mlhip::fail_logic(std::string("HIP backend: ") + (msg)); } while (0)

	inline Context* get(mlContext_t context)
	{
		if (context == nullptr)
			fail_logic("HIP backend: null context");
		return reinterpret_cast<Context*>(context);
	}
	inline hipStream_t stream_of(mlContext_t context)
	{
		return get(context)->stream;
	}
	/* returns device scratch of at least `bytes` bytes; grows by reallocating after the stream has drained */
	void* get_workspace(mlContext_t context, size_t bytes);
	/* winograd.hip; called once per context creation with that device current: looks up, per device, the address of the static device
	 * array behind hip_winograd_layer_forward_static and raises the dynamic-LDS limit of the kernels that run from it */
	void prepare_static_memory(int device_index);
	/* number of compute units of the current device (cached per device) */
	int device_compute_units();
	/* makes sure a kernel may be launched with `bytes` of dynamic LDS on the current device (requests above the 64 KB default raise the
	 * kernel's limit; the largest size granted so far is remembered per device and kernel) */
	void ensure_dynamic_lds(const void *kernel, int bytes);

	inline int size_of(mlDataType_t dtype)
	{
		switch (dtype)
		{
			case DTYPE_FLOAT8:
			case DTYPE_UINT8:
			case DTYPE_INT8:
				return 1;
			case DTYPE_FLOAT16:
			case DTYPE_INT16:
				return 2;
			case DTYPE_FLOAT32:
			case DTYPE_INT32:
				return 4;
			case DTYPE_FLOAT64:
				return 8;
			default:
				return 0;
		}
	}
	inline size_t volume(const mlShape_t &s)
	{
		if (s.rank == 0)
			return 0;
		size_t result = 1;
		for (int i = 0; i < s.rank; i++)
			result *= static_cast<size_t>(s.dim[i]);
		return result;
	}
	inline size_t volume(const mlTensor_t &t)
	{
		if (t.rank == 0)
			return 0;
		size_t result = 1;
		for (int i = 0; i < t.rank; i++)
			result *= static_cast<size_t>(t.dim[i]);
		return result;
	}
	inline int last_dim(const mlTensor_t &t)
	{
		return (t.rank == 0) ? 0 : t.dim[t.rank - 1];
	}
	inline int last_dim(const mlShape_t &s)
	{
		return (s.rank == 0) ? 0 : s.dim[s.rank - 1];
	}
	inline mlShape_t shape_of(const mlTensor_t &t)
	{
		mlShape_t s;
		s.rank = t.rank;
		for (int i = 0; i < 6; i++)
			s.dim[i] = t.dim[i];
		return s;
	}
	inline mlTensor_t make_tensor(const void *data, mlDataType_t dtype, const mlShape_t &shape)
	{
		mlTensor_t t;
		t.data = const_cast<void*>(data);
		t.dtype = dtype;
		t.rank = shape.rank;
		for (int i = 0; i < 6; i++)
			t.dim[i] = shape.dim[i];
		return t;
	}
	inline bool is_transpose(char op)
	{
		if (op == 't' || op == 'T')
			return true;
		if (op == 'n' || op == 'N')
			return false;
		fail_logic("HIP backend: matrix op must be one of 'n', 'N', 't', 'T'");
	}
	template<typename T>
	inline T* ptr(const mlTensor_t &t)
	{
		return reinterpret_cast<T*>(t.data);
	}
	inline int ceil_div(int a, int b)
	{
		return (a + b - 1) / b;
	}
} /* namespace mlhip */

/*
 * Exports hip_<name> a second time as cuda_<name>, the symbol minml's unmodified dispatcher calls for a device backend.
 * An alias shares the definition, so both names have one address and one behaviour. Host pass only.
 */
#if defined(__HIP_DEVICE_COMPILE__)
#define MLHIP_ALSO_AS_CUDA(name)
#else
#define MLHIP_ALSO_AS_CUDA(name) extern "C" __typeof__(hip_##name) cuda_##name __attribute__((alias("hip_" #name)));
#endif

#endif /* MINML_AMD_COMMON_HPP_ */
