/*
 * cabi_errors.cpp — error behaviour of the C-ABI, exercised from C++ because the library reports failures the reference's way:
 * C++ exceptions crossing the extern "C" boundary (reference: src/backend/cuda_dummy_backend.cpp:25-27 throws NotImplemented,
 * src/backend/cpu/winograd/winograd_runtime.cpp:516 throws std::runtime_error("No suitable Winograd transform runtime"),
 * src/backend/cpu/dispatcher.cpp:61 throws std::logic_error). Every case fails during argument checking, before any device call, so the
 * program runs on a machine without a GPU. Prints one line per case and exits 0 when all behaved.
 */
#include "../include/minml_hip_backend.h"

#include <cstdio>
#include <cstring>
#include <functional>
#include <stdexcept>
#include <string>

extern "C"
{
	void cuda_batchnorm_forward(); /* a symbol outside the path: defined, throws */
	void cuda_winograd_input_transform(mlContext_t, int, const mlTensor_t, mlTensor_t);
	void cuda_gemm_v2(mlContext_t, char, char, float, const mlTensor_t, const mlTensor_t, float, mlTensor_t);
}

static mlTensor_t tensor(void *data, mlDataType_t dtype, int rank, int d0 = 0, int d1 = 0, int d2 = 0, int d3 = 0)
{
	mlTensor_t t;
	std::memset(&t, 0, sizeof(t));
	t.data = data;
	t.dtype = dtype;
	t.rank = rank;
	t.dim[0] = d0;
	t.dim[1] = d1;
	t.dim[2] = d2;
	t.dim[3] = d3;
	return t;
}
static mlShape_t shape(int rank, int d0 = 0, int d1 = 0, int d2 = 0, int d3 = 0)
{
	mlShape_t s;
	std::memset(&s, 0, sizeof(s));
	s.rank = rank;
	s.dim[0] = d0;
	s.dim[1] = d1;
	s.dim[2] = d2;
	s.dim[3] = d3;
	return s;
}

static int failures = 0;

template<typename E>
static void expect_throw(const char *name, const std::function<void()> &f, const char *needle)
{
	try
	{
		f();
		std::printf("FAIL %s: no exception\n", name);
		failures++;
	} catch (const E &e)
	{
		if (needle != nullptr && std::string(e.what()).find(needle) == std::string::npos)
		{
			std::printf("FAIL %s: message '%s' lacks '%s'\n", name, e.what(), needle);
			failures++;
		}
		else
			std::printf("OK %s: %s\n", name, e.what());
	} catch (...)
	{
		std::printf("FAIL %s: wrong exception type\n", name);
		failures++;
	}
}

int main()
{
	static float buffer[36 * 64];
	/* tile 5 on a 3x3 kernel: 49 matrices */
	expect_throw<std::runtime_error>("winograd tile 5", [&]()
	{	hip_winograd_input_transform(nullptr, 5, tensor(buffer, DTYPE_FLOAT32, 4, 1, 5, 5, 2), tensor(buffer, DTYPE_FLOAT32, 3, 49, 1, 2));}, "No suitable Winograd transform runtime");
	/* int8 is not a Winograd type */
	expect_throw<std::runtime_error>("winograd int8", [&]()
	{	hip_winograd_input_transform(nullptr, 4, tensor(buffer, DTYPE_INT8, 4, 1, 4, 4, 2), tensor(buffer, DTYPE_INT8, 3, 36, 1, 2));}, "No suitable Winograd transform runtime");
	/* the same through the reference's symbol name */
	expect_throw<std::runtime_error>("cuda_ alias", [&]()
	{	cuda_winograd_input_transform(nullptr, 5, tensor(buffer, DTYPE_FLOAT32, 4, 1, 5, 5, 2), tensor(buffer, DTYPE_FLOAT32, 3, 49, 1, 2));}, "No suitable Winograd transform runtime");
	/* wrong matrices shape */
	expect_throw<std::logic_error>("winograd matrices shape", [&]()
	{	hip_winograd_input_transform(nullptr, 4, tensor(buffer, DTYPE_FLOAT32, 4, 1, 4, 4, 2), tensor(buffer, DTYPE_FLOAT32, 3, 36, 7, 2));}, "matrices must be");
	/* GEMM argument errors */
	expect_throw<std::logic_error>("gemm bad op", [&]()
	{	hip_gemm(nullptr, DTYPE_FLOAT32, shape(2, 4, 4), buffer, shape(2, 4, 4), buffer, shape(2, 4, 4), buffer, 'x', 'n', 1.0f, 0.0f);}, "matrix op");
	expect_throw<std::logic_error>("gemm inner dims", [&]()
	{	hip_gemm(nullptr, DTYPE_FLOAT32, shape(2, 4, 4), buffer, shape(2, 4, 5), buffer, shape(2, 4, 6), buffer, 'n', 't', 1.0f, 0.0f);}, "inner dimensions");
	expect_throw<std::logic_error>("gemm rank", [&]()
	{	hip_gemm(nullptr, DTYPE_FLOAT32, shape(2, 4, 4), buffer, shape(4, 1, 1, 4, 4), buffer, shape(2, 4, 4), buffer, 'n', 't', 1.0f, 0.0f);}, "rank");
	expect_throw<std::logic_error>("int8 gemm alpha", [&]()
	{	cuda_gemm_v2(nullptr, 'n', 't', 2.0f, tensor(buffer, DTYPE_INT8, 2, 4, 16), tensor(buffer, DTYPE_INT8, 2, 4, 16), 0.0f, tensor(buffer, DTYPE_INT32, 2, 4, 4));}, "alpha = 1");
	/* convolution argument errors */
	expect_throw<std::logic_error>("conv filters", [&]()
	{	hip_convolution_implicit_gemm_forward(nullptr, DTYPE_FLOAT16, shape(4, 1, 5, 5, 8), shape(4, 4, 3, 3, 16), buffer, buffer, buffer, nullptr, nullptr, ACTIVATION_RELU);}, "input filters");
	expect_throw<std::logic_error>("conv dtype", [&]()
	{	hip_convolution_implicit_gemm_forward(nullptr, DTYPE_INT8, shape(4, 1, 5, 5, 8), shape(4, 4, 3, 3, 8), buffer, buffer, buffer, nullptr, nullptr, ACTIVATION_RELU);}, "unsupported data type");
	expect_throw<std::logic_error>("convert", [&]()
	{	hip_convert_type(nullptr, buffer, DTYPE_INT32, buffer + 64, DTYPE_FLOAT32, 4);}, "unsupported conversion");
	/* attention argument errors */
	expect_throw<std::logic_error>("attention heads", [&]()
	{	hip_multi_head_attention_forward(nullptr, shape(4, 1, 4, 4, 96), shape(0), shape(0), DTYPE_FLOAT32, buffer, buffer, nullptr, nullptr, nullptr, nullptr, 5, false);}, "divisible by the number of heads");
	expect_throw<std::logic_error>("attention table", [&]()
	{	hip_multi_head_attention_forward(nullptr, shape(4, 1, 4, 4, 96), shape(3, 4, 5, 5), shape(0), DTYPE_FLOAT32, buffer, buffer, buffer, nullptr, nullptr, nullptr, 4, false);}, "position table");
	expect_throw<std::runtime_error>("attention training", [&]()
	{	hip_multi_head_attention_forward(nullptr, shape(4, 1, 4, 4, 96), shape(0), shape(0), DTYPE_FLOAT32, buffer, buffer, nullptr, nullptr, nullptr, buffer, 4, false);}, "inference only");
	expect_throw<std::logic_error>("rmsnorm dtype", [&]()
	{	hip_rmsnorm_forward(nullptr, shape(2, 4, 8), DTYPE_INT8, buffer, buffer, nullptr);}, "unsupported data type");
	/* valid arguments but no context */
	expect_throw<std::logic_error>("null context", [&]()
	{	hip_winograd_input_transform(nullptr, 4, tensor(buffer, DTYPE_FLOAT32, 4, 1, 4, 4, 2), tensor(buffer, DTYPE_FLOAT32, 3, 36, 1, 2));}, "null context");
	/* no such device */
	expect_throw<std::logic_error>("create_context(12345)", [&]()
	{	hip_create_context(12345);}, "no such device");
	/* outside the path */
	expect_throw<std::logic_error>("stub", [&]()
	{	cuda_batchnorm_forward();}, "not implemented");

	/* calls that must NOT throw without a device: empty work and identity queries */
	try
	{
		hip_winograd_input_transform(nullptr, 4, tensor(nullptr, DTYPE_FLOAT32, 4, 0, 4, 4, 2), tensor(nullptr, DTYPE_FLOAT32, 3, 36, 0, 2));
		hip_gemm(nullptr, DTYPE_FLOAT32, shape(2, 0, 4), nullptr, shape(2, 0, 8), nullptr, shape(2, 4, 8), buffer, 'n', 't', 1.0f, 0.0f);
		(void) hip_get_number_of_devices();
		(void) hip_supports_type(12345, DTYPE_FLOAT16);
		hip_rmsnorm_forward(nullptr, shape(2, 0, 8), DTYPE_FLOAT32, nullptr, nullptr, nullptr);
		if (hip_multi_head_attention_get_workspace_size(shape(4, 256, 15, 15, 768), shape(3, 8, 29, 32), 8, false) != 0)
			throw std::runtime_error("inference attention asks for workspace");
		hip_destroy_context(nullptr);
		hip_destroy_event(nullptr);
		hip_free(nullptr);
		std::printf("OK no-throw cases\n");
	} catch (const std::exception &e)
	{
		std::printf("FAIL no-throw cases: %s\n", e.what());
		failures++;
	}

	std::printf("%s\n", failures == 0 ? "ALL OK" : "FAILED");
	return failures == 0 ? 0 : 1;
}
