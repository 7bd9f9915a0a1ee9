/*
 * dropin_graph.cpp — the reference's own Graph / Conv2D / dispatcher code running on the HIP backend, unmodified.
 *
 * The program is compiled against the reference's headers and linked with the reference's src/core, src/layers, src/graph, src/training,
 * src/utils and CPU backend objects plus libminml_hip.so, WITHOUT src/backend/cuda_dummy_backend.cpp: every cuda_* symbol that the
 * reference's dispatcher calls for DeviceType::CUDA (src/core/math.cpp, ml_memory.cpp, Context.cpp, Event.cpp, Device.cpp) resolves to
 * the HIP library (link recipe: oracle/Makefile, target `dropin`; the reference swaps backends the same way, CMakeLists.txt:60-65).
 *
 *   dropin_graph link                       exits 0: proves that the executable links and loads (no GPU needed)
 *   dropin_graph run <batch> <channels> <blocks> [verbose]
 *       builds the residual network of benchmark configuration 1 as a reference Graph (stem 3x3 conv, `blocks` residual blocks of two 3x3
 *       convolutions with an Add, 1x1 policy head), applies the reference's FoldAdd pass, runs Graph::predict on Device::cpu() and on
 *       Device::cuda(0) (= the HIP backend) in fp32 and, after Graph::convertTo(FLOAT16), in fp16, and prints the max-abs relative
 *       differences of every layer's output and of the head (`verbose`: one line per layer). Exit code 1 when a layer exceeds 1e-4 in
 *       fp32 or 1e-2 in fp16.
 *   dropin_graph time <batch> <channels> <blocks> <fp32|fp16> <seconds> [warm-up passes]
 *       the same graph on Device::cuda(0) only, timed the way the reference's launcher times a network (launcher/minml.cpp:3924-3936):
 *       Graph::predict followed by Context::synchronize, repeated until `seconds` have passed; prints "time = ..s, repeats = .., n/s = .."
 *       (n/s = positions per second). This is the throughput an unchanged minml gets from the backend: three calls per 3x3 layer.
 */
#include <minml/core/Context.hpp>
#include <minml/core/Device.hpp>
#include <minml/core/Tensor.hpp>
#include <minml/graph/Graph.hpp>
#include <minml/graph/GraphNode.hpp>
#include <minml/graph/graph_optimizers.hpp>
#include <minml/layers/Add.hpp>
#include <minml/layers/Conv2D.hpp>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <string>
#include <vector>

using namespace ml;

static std::vector<float> to_host_floats(const Context &context, const Tensor &tensor)
{
	Tensor out(tensor.shape(), tensor.dtype(), Device::cpu());
	out.copyFrom(context, tensor);
	context.synchronize();
	if (out.dtype() != DataType::FLOAT32)
		out.convertTo(Context(Device::cpu()), DataType::FLOAT32);
	std::vector<float> result(out.volume());
	std::memcpy(result.data(), out.data(), result.size() * sizeof(float));
	return result;
}
/* one Graph::predict; returns the output tensor of every node (the last one is the head) */
static std::vector<std::vector<float>> node_outputs(Graph &graph, int batch, const std::vector<float> &planes)
{
	Tensor &input = graph.getInput();
	/* Tensor::copyFrom converts nothing: upload in the graph's storage type through a host tensor of that type */
	Tensor staged(input.shape(), "float32", Device::cpu());
	std::memcpy(staged.data(), planes.data(), planes.size() * sizeof(float));
	if (input.dtype() != DataType::FLOAT32)
		staged.convertTo(Context(Device::cpu()), input.dtype());
	input.copyFrom(graph.context(), staged);
	graph.predict(batch);
	graph.context().synchronize();
	std::vector<std::vector<float>> result;
	for (int i = 0; i < graph.numberOfNodes(); i++)
		result.push_back(to_host_floats(graph.context(), graph.getNode(i).getOutputTensor()));
	return result;
}
/* Conv2D carries its Winograd-transformed weights along in Graph::moveTo (src/layers/Conv2D.cpp:186-197); dropping the cache makes
 * every device transform its own (the CPU backend of a non-trainable layer would have cached matrices for 5x5 tiles, Conv2D.cpp:461) */
static void move_graph(Graph &graph, Device device)
{
	graph.moveTo(device);
	for (int i = 0; i < graph.numberOfNodes(); i++)
		if (Conv2D *conv = dynamic_cast<Conv2D*>(&graph.getNode(i).getLayer()))
			conv->invalidateWeightsCache();
}
static double relative_difference(const std::vector<float> &a, const std::vector<float> &b)
{
	double diff = 0.0, scale = 1.0e-6;
	for (size_t i = 0; i < a.size(); i++)
	{
		diff = std::max(diff, static_cast<double>(std::fabs(a[i] - b[i])));
		scale = std::max(scale, static_cast<double>(std::fabs(b[i])));
	}
	return diff / scale;
}

/* the residual network of the benchmark configurations as a reference Graph, after the reference's FoldAdd pass */
static void build_network(Graph &graph, int batch, int board, int planes, int channels, int blocks)
{
	GraphNodeID x = graph.addInput(Shape( { batch, board, board, planes }));
	x = graph.add(Conv2D(channels, 3, "relu"), x);
	for (int i = 0; i < blocks; i++)
	{
		GraphNodeID y = graph.add(Conv2D(channels, 3, "relu"), x);
		y = graph.add(Conv2D(channels, 3, "linear"), y);
		x = graph.add(Add("relu"), { x, y }); /* skip connection first: FoldAdd hands Add's input 0 to the convolution (graph_optimizers.cpp:211) */
	}
	x = graph.add(Conv2D(1, 1, "linear"), x);
	graph.addOutput(x);
	graph.init(); /* the reference's own initialiser; the same parameters then serve both devices */
	/* left trainable on purpose: the CPU backend then takes its F(4x4, 3x3) kernels, the algorithm of the device branch and of the
	 * benchmark configurations; a non-trainable layer switches the CPU side alone to 5x5 tiles (Conv2D.cpp:461) */
	const int nodes_before = graph.numberOfNodes();
	FoldAdd().optimize(graph);
	std::printf("graph: %d nodes, %d after FoldAdd\n", nodes_before, graph.numberOfNodes());
}
static std::vector<float> bernoulli_planes(size_t count)
{
	std::vector<float> input(count);
	uint64_t state = 0x9e3779b97f4a7c15ull;
	for (size_t i = 0; i < input.size(); i++)
	{ /* Bernoulli(0.3) planes from a 64-bit LCG */
		state = state * 6364136223846793005ull + 1442695040888963407ull;
		input[i] = ((state >> 40) < static_cast<uint64_t>(0.3 * (1ull << 24))) ? 1.0f : 0.0f;
	}
	return input;
}
static double seconds_now()
{
	return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
static int time_mode(int argc, char **argv)
{
	const int batch = std::atoi(argv[2]), channels = std::atoi(argv[3]), blocks = std::atoi(argv[4]);
	const bool half = std::string(argv[5]) == "fp16";
	const double budget = std::atof(argv[6]);
	const int warmup = (argc >= 8) ? std::atoi(argv[7]) : 3;
	const int board = 15, planes = 32;
	if (batch <= 0 || channels <= 0 || blocks < 0 || budget <= 0.0 || (!half && std::string(argv[5]) != "fp32"))
	{
		std::fprintf(stderr, "time: bad arguments\n");
		return 2;
	}
	if (Device::numberOfCudaDevices() < 1)
	{
		std::fprintf(stderr, "no device behind the cuda_* entry points\n");
		return 3;
	}
	Graph graph;
	build_network(graph, batch, board, planes, channels, blocks);
	if (half)
		graph.convertTo(DataType::FLOAT16);
	move_graph(graph, Device::cuda(0));
	const std::vector<float> planes_host = bernoulli_planes(static_cast<size_t>(batch) * board * board * planes);
	Tensor &input = graph.getInput();
	Tensor staged(input.shape(), "float32", Device::cpu());
	std::memcpy(staged.data(), planes_host.data(), planes_host.size() * sizeof(float));
	if (half)
		staged.convertTo(Context(Device::cpu()), input.dtype());
	input.copyFrom(graph.context(), staged);
	for (int i = 0; i < warmup; i++)
	{
		graph.predict(batch);
		graph.context().synchronize();
	}
	const double start = seconds_now();
	int repeats = 0;
	do
	{ /* as the reference's launcher: one predict, one synchronize, until the time is up */
		graph.predict(batch);
		graph.context().synchronize();
		repeats++;
	} while (seconds_now() - start < budget);
	const double elapsed = seconds_now() - start;
	const std::vector<float> head = to_host_floats(graph.context(), graph.getOutput(0));
	double norm = 0.0;
	for (float v : head)
		norm += std::fabs(v);
	std::printf("time = %.4fs, repeats = %d, n/s = %.1f, ms per predict = %.4f, mean |logit| = %.6f (%s, batch %d, %d blocks x %d channels, on %s)\n", elapsed,
			repeats, batch * repeats / elapsed, 1.0e3 * elapsed / repeats, norm / head.size(), half ? "fp16" : "fp32", batch, blocks, channels,
			Device::cuda(0).toString().c_str());
	return std::isfinite(norm) ? 0 : 1;
}

int main(int argc, char **argv)
{
	if (argc >= 2 && std::string(argv[1]) == "link")
	{
		std::printf("linked: the reference's dispatcher sees %d device(s) behind its cuda_* entry points\n", Device::numberOfCudaDevices());
		return 0;
	}
	if (argc >= 7 && std::string(argv[1]) == "time")
	{
		try
		{
			return time_mode(argc, argv);
		} catch (std::exception &e)
		{
			std::fprintf(stderr, "exception: %s\n", e.what());
			return 4;
		}
	}
	const bool verbose = (argc == 6 && std::string(argv[5]) == "verbose");
	if ((argc != 5 && !verbose) || std::string(argv[1]) != "run")
	{
		std::fprintf(stderr, "usage: %s link | run <batch> <channels> <blocks> [verbose] | time <batch> <channels> <blocks> <fp32|fp16> <seconds> [warm-up]\n", argv[0]);
		return 2;
	}
	try
	{
		const int batch = std::atoi(argv[2]), channels = std::atoi(argv[3]), blocks = std::atoi(argv[4]);
		const int board = 15, planes = 32;
		if (Device::numberOfCudaDevices() < 1)
		{
			std::fprintf(stderr, "no device behind the cuda_* entry points\n");
			return 3;
		}
		Graph graph;
		build_network(graph, batch, board, planes, channels, blocks);
		const std::vector<float> input = bernoulli_planes(static_cast<size_t>(batch) * board * board * planes);

		bool ok = true;
		for (int pass = 0; pass < 2; pass++)
		{
			const bool half = (pass == 1);
			if (half)
			{
				move_graph(graph, Device::cpu());
				graph.convertTo(DataType::FLOAT16);
			}
			const std::vector<std::vector<float>> on_cpu = node_outputs(graph, batch, input);
			move_graph(graph, Device::cuda(0));
			const std::vector<std::vector<float>> on_device = node_outputs(graph, batch, input);
			const double limit = half ? 1.0e-2 : 1.0e-4;
			double worst = 0.0;
			for (size_t n = 1; n < on_cpu.size(); n++)
			{
				const double err = relative_difference(on_device[n], on_cpu[n]);
				worst = std::max(worst, err);
				if (verbose || !(err <= limit))
					std::printf("  %s node %2d (%s): %.3e\n", half ? "fp16" : "fp32", static_cast<int>(n), graph.getNode(n).getLayer().name().c_str(), err);
			}
			const double head = relative_difference(on_device.back(), on_cpu.back());
			std::printf("%s: Graph::predict on %s vs Device::cpu(): max-abs relative difference %.3e at the head, %.3e worst layer (limit %.0e)\n",
					half ? "fp16" : "fp32", Device::cuda(0).toString().c_str(), head, worst, limit);
			if (!(worst <= limit))
				ok = false;
		}
		std::printf(ok ? "dropin ok\n" : "dropin FAILED\n");
		return ok ? 0 : 1;
	} catch (std::exception &e)
	{
		std::fprintf(stderr, "exception: %s\n", e.what());
		return 4;
	}
}
