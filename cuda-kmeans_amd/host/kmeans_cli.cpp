/*
 * k-means command-line harness for the MI355X kernels.
 *
 * Keeps the behaviour of the reference's driver (experimental/k-means/k-means/k-means.cpp): the same option
 * names with k/M/G suffixes (:298-327), algorithms picked by name from a map (:66-81,129-145), initialize()
 * and run() timed with a wall clock, stdout = "<ms per iteration> <ns per input float>" and prose on stderr
 * (:147-169), --verify against the serial algorithm (:171-182), exit code 1 for bad arguments and 2 for
 * run-time errors (:332-350). Device algorithms are named hip_*; the reference's cuda_* names are accepted
 * as aliases of their counterparts. Additions: --dataset / --config / --init select the seeded benchmark
 * data sets with first-k initial centroids, --serialThreads speeds the serial yardstick up without
 * changing a bit of its results, --json prints a machine-readable report with the assignment / update
 * split and the mismatch classification.
 */
#include "cli_args.hpp"
#include "datasets.hpp"
#include "hip_kmeans.hpp"
#include "kmeans_interface.hpp"
#include "layouts.hpp"
#include "metrics.hpp"
#include "serial_kmeans.hpp"

#include <chrono>
#include <cstdio>
#include <cstring>
#include <cstdint>
#include <iostream>
#include <map>
#include <vector>
#include <memory>
#include <string>

namespace {

class Stopwatch
{
	std::chrono::steady_clock::time_point mStart;
	double mMs = 0.0;
public:
	void start() { mStart = std::chrono::steady_clock::now(); }
	void stop() { mMs = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - mStart).count(); }
	double getMiliseconds() const { return mMs; }
};

/* raw little-endian dump of a result vector (--dump): <prefix>.means.f32 (.f64 with --double) / <prefix>.assignment.u32 */
template<typename T>
void dumpVector(const std::string& path, const std::vector<T>& v)
{
	std::FILE* f = std::fopen(path.c_str(), "wb");
	if (!f) throw std::runtime_error("Cannot open '" + path + "' for writing.");
	const std::size_t written = std::fwrite(v.data(), sizeof(T), v.size(), f);
	std::fclose(f);
	if (written != v.size()) throw std::runtime_error("Short write to '" + path + "'.");
}

/* reference names -> names of this build */
std::string canonicalAlgorithm(const std::string& name)
{
	static const std::map<std::string, std::string> aliases = {
		{ "cuda_base", "hip_base" }, { "cuda_base_shm", "hip_base_shm" }, { "cuda_best", "hip_best" },
		{ "cuda_cached_fixed", "hip_lds_fma" }, { "cuda_cached_regs", "hip_mfma" },
		{ "cuda_cached_means", "hip_lds_fma" }, /* CachedAllMeansAssignmentKernel (k-means.cpp:72, kernels.cu:328-410): all centroids in LDS, which is what the LDS/FMA variant does */
		{ "cuda_fused_fixed", "hip_fused" }, { "cuda_fused_regs", "hip_fused" },
	};
	auto it = aliases.find(name);
	return it == aliases.end() ? name : it->second;
}

void getHipExecParameters(const ProgramArguments& args, HipExecParameters& exec)
{
	exec.blockSize = (unsigned int)args.getInt("cudaBlockSize");
	exec.blockCount = (unsigned int)args.getInt("cudaBlockCount");
	exec.sharedMemorySize = args.isPresent("cudaSharedMemorySize") ? (unsigned int)args.getInt("cudaSharedMemorySize") : 0; /* 0 = device maximum */
	exec.privatizedCopies = (std::uint32_t)args.getInt("privatizedCopies");
	exec.itemsPerThread = (std::uint32_t)args.getInt("itemsPerThread");
	exec.regsCache = (std::uint32_t)args.getInt("regsCache");
}

/*
 * The reference's launch parameters (k-means.cpp:318-326) shape the launches of the kernels that have that freedom:
 * hip_base (one lane per point) and the global-atomic update behind it. The tuned kernels fix their own work-group
 * shape (8 wavefronts around the LDS-resident centroids, 16 around a sorted chunk, the MFMA tile as register tile), so
 * a value given for one of these options changes nothing there: say so instead of leaving a parameter sweep to wonder
 * why its times do not move.
 */
void warnIgnoredLaunchParameters(const ProgramArguments& args, const std::string& algoName)
{
	static const std::map<std::string, std::vector<const char*>> ignored = {
		{ "hip_base", { "regsCache" } },
		{ "hip_base_shm", { "regsCache", "privatizedCopies" } },
		{ "hip_lds_fma", { "cudaBlockSize", "itemsPerThread", "regsCache", "privatizedCopies" } },
		{ "hip_mfma", { "cudaBlockSize", "itemsPerThread", "regsCache", "privatizedCopies" } },
		{ "hip_mfma_bf16", { "cudaBlockSize", "itemsPerThread", "regsCache", "privatizedCopies" } },
		{ "hip_best", { "cudaBlockSize", "itemsPerThread", "regsCache", "privatizedCopies" } },
		{ "hip_best_serial_order", { "cudaBlockSize", "itemsPerThread", "regsCache", "privatizedCopies" } },
		{ "hip_fused", { "cudaBlockSize", "itemsPerThread", "regsCache", "privatizedCopies" } },
	};
	auto it = ignored.find(algoName);
	if (it == ignored.end()) return;
	for (const char* name : it->second)
		if (args.isPresent(name))
			std::cerr << "Warning: --" << name << " is ignored by " << algoName << " (its kernels fix their own launch shape)." << std::endl;
}

/* capability checks of the reference's getCudaExecParameters (k-means.cpp:27-41), once a device algorithm is chosen */
void checkDevice(const HipExecParameters& exec)
{
	requireDevice();
	kmx_props props;
	KMX_CHECK(kmx_device_props(&props));
	if (exec.blockSize > props.max_threads_per_block)
		throw std::runtime_error("Requested block size (" + std::to_string(exec.blockSize) + ") exceeds device capabilities ("
			+ std::to_string(props.max_threads_per_block) + ").");
	if (exec.sharedMemorySize > props.lds_bytes_per_block)
		throw std::runtime_error("Requested shared memory per block (" + std::to_string(exec.sharedMemorySize) + ") exceeds device capabilities ("
			+ std::to_string(props.lds_bytes_per_block) + ").");
	std::cerr << "HIP device #0 selected: " << props.arch << ", " << props.compute_units << " CUs ("
		<< props.lds_bytes_per_block / 1024 << "kB LDS per work-group)" << std::endl;
}

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS, class METRIC>
void run_assignment(const ProgramArguments& args, std::vector<F>& data, std::vector<F>& means)
{
	const std::size_t dim = (std::size_t)args.getInt("dim"), k = (std::size_t)args.getInt("k"), n = (std::size_t)args.getInt("N");
	const std::string algoName = canonicalAlgorithm(args.getString("algorithm"));
	const int threads = (int)args.getInt("serialThreads");

	HipExecParameters exec;
	getHipExecParameters(args, exec);

	using map_t = std::map<std::string, std::unique_ptr<IAssignmentAlgorithm<F, IDX_T>>>;
	map_t algorithms;
	algorithms["serial"].reset(new SerialAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>(threads));
	algorithms["hip_base"].reset(new HipAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, BaseAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>(exec));
	algorithms["hip_lds_fma"].reset(new HipAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, LdsFmaAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>(exec));
	algorithms["hip_mfma"].reset(new HipAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, MfmaAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>(exec));
	algorithms["hip_mfma_bf16"].reset(new HipAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, MfmaBf16AssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>(exec));
	algorithms["hip_best"].reset(new HipAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, BestCachedAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>(exec));

	auto it = algorithms.find(algoName);
	if (it == algorithms.end()) throw std::runtime_error("Unkown algorithm '" + algoName + "'.");
	warnIgnoredLaunchParameters(args, algoName);
	if (algoName != "serial") checkDevice(exec);
	std::cerr << "Selected assignment-only algorithm: " << algoName << std::endl;
	auto algorithm = std::move(it->second);

	Stopwatch stopwatch;
	std::cerr << "Initializing ... "; std::cerr.flush();
	stopwatch.start();
	algorithm->initialize(dim, k, n, data, means);
	stopwatch.stop();
	std::cerr << stopwatch.getMiliseconds() << " ms" << std::endl;

	std::cerr << "Running (assignment only) ... "; std::cerr.flush();
	stopwatch.start();
	algorithm->run();
	stopwatch.stop();
	std::cout << stopwatch.getMiliseconds(); std::cout.flush();
	std::cerr << " ms (which is"; std::cerr.flush();
	std::cout << " " << (stopwatch.getMiliseconds() * 1000000.0 / (double)(dim * n)); std::cout.flush();
	std::cerr << " ns/input float)"; std::cerr.flush();
	std::cout << std::endl;

	if (args.getBool("verify") && algoName != "serial") {
		std::cerr << "Verifying results ... "; std::cerr.flush();
		SerialAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC> base(threads);
		base.initialize(dim, k, n, data, means);
		base.run();
		if (verify_assignment<IDX_T>(algorithm->getAssignment(), base.getAssignment(), n) == 0) std::cerr << "OK" << std::endl;
		else {
			auto report = classify_mismatches<F, IDX_T, LAYOUT, LAYOUT_MEANS>(algorithm->getAssignment(), base.getAssignment(), data, means, dim, k, n);
			std::cerr << "FAILED (" << report.mismatches << " mismatches, " << report.nearTies << " of them near-ties below 1e-5)" << std::endl;
		}
	}
	algorithm->cleanup();
}

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS, class METRIC>
void run_kmeans(const ProgramArguments& args, std::vector<F>& data, std::vector<F>& means)
{
	const std::size_t dim = (std::size_t)args.getInt("dim"), k = (std::size_t)args.getInt("k"), n = (std::size_t)args.getInt("N");
	std::size_t iters = (std::size_t)args.getInt("iterations");
	const std::string algoName = canonicalAlgorithm(args.getString("algorithm"));
	const int threads = (int)args.getInt("serialThreads");
	const bool json = args.getBool("json");

	HipExecParameters exec;
	getHipExecParameters(args, exec);

	const bool graph = args.getBool("graph");
	using Base = BaseAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>;
	using Best = BestCachedAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>;
	using Mfma = MfmaAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>;
	using MfmaBf16 = MfmaBf16AssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>;
	using Point = UpdateAtomicPointKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS>;
	using Shm = UpdateAtomicShmKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS>;
	using Ordered = UpdateSerialOrderKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS>;
	using map_t = std::map<std::string, std::unique_ptr<IKMeansAlgorithm<F, IDX_T>>>;
	map_t algorithms;
	algorithms["serial"].reset(new SerialKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>(threads));
	algorithms["hip_base"].reset(new HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, Base, Point>(exec, json, graph));
	algorithms["hip_base_shm"].reset(new HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, Base, Shm>(exec, json, graph));
	algorithms["hip_mfma"].reset(new HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, Mfma, Shm>(exec, json, graph));
	algorithms["hip_mfma_bf16"].reset(new HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, MfmaBf16, Shm>(exec, json, graph));
	algorithms["hip_best"].reset(new HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, Best, Shm>(exec, json, graph));
	/* the fastest assignment with the update that adds in the serial order: the whole run has the bits of `serial` */
	algorithms["hip_best_serial_order"].reset(new HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, Best, Ordered>(exec, json, graph));
	algorithms["hip_fused"].reset(new HipFusedKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>(exec));

	auto it = algorithms.find(algoName);
	if (it == algorithms.end()) throw std::runtime_error("Unkown algorithm '" + algoName + "'.");
	warnIgnoredLaunchParameters(args, algoName);
	if (algoName != "serial") checkDevice(exec);
	std::cerr << "Selected k-means algorithm: " << algoName << std::endl;
	auto algorithm = std::move(it->second);

	Stopwatch stopwatch;
	std::cerr << "Initializing ... "; std::cerr.flush();
	stopwatch.start();
	algorithm->initialize(dim, k, n, iters, data, means);
	stopwatch.stop();
	const double initMs = stopwatch.getMiliseconds();
	std::cerr << initMs << " ms" << std::endl;

	std::cerr << "Running (" << iters << " iterations) ... "; std::cerr.flush();
	stopwatch.start();
	algorithm->run();
	stopwatch.stop();
	if (algorithm->getIterations() != iters) {
		iters = algorithm->getIterations();
		std::cerr << "[stopped after " << iters << " iters.] ";
	}
	const double msPerIter = stopwatch.getMiliseconds() / (double)iters;
	const double nsPerFloat = stopwatch.getMiliseconds() * 1000000.0 / (double)(iters * dim * n);
	if (!json) { std::cout << msPerIter; std::cout.flush(); }
	std::cerr << " ms/iter (which is"; std::cerr.flush();
	if (!json) { std::cout << " " << nsPerFloat; std::cout.flush(); }
	std::cerr << " ns/input float)"; std::cerr.flush();
	if (!json) std::cout << std::endl; else std::cerr << std::endl;

	std::size_t errors = 0, mismatches = 0;
	double centroidErr = 0.0;
	bool verified = false, identical = false;
	if (args.getBool("verify") && algoName != "serial") {
		std::cerr << "Verifying results ... "; std::cerr.flush();
		SerialKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC> base(threads);
		base.initialize(dim, k, n, iters, data, means);
		base.run();
		if (algoName == "hip_fused") {
			/* the fused algorithm reports the assignment against its FINAL centroids (cuda.hpp:199-221), the serial
			 * algorithm the one its last iteration used: compare with a serial assignment pass over the same centroids */
			SerialAssignmentAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC> last(threads);
			last.initialize(dim, k, n, data, algorithm->getMeans());
			last.run();
			mismatches = verify_assignment<IDX_T>(algorithm->getAssignment(), last.getAssignment(), n);
		}
		else mismatches = verify_assignment<IDX_T>(algorithm->getAssignment(), base.getAssignment(), n);
		errors = mismatches + verify_means<F, LAYOUT_MEANS>(algorithm->getMeans(), base.getMeans(), dim, k);
		centroidErr = centroid_error<F, LAYOUT_MEANS>(algorithm->getMeans(), base.getMeans(), dim, k);
		verified = true;
		/* the same bits as the serial run: every assignment equal and the centroid buffers equal byte for byte */
		identical = mismatches == 0 && algorithm->getMeans().size() == base.getMeans().size()
			&& std::memcmp(algorithm->getMeans().data(), base.getMeans().data(), base.getMeans().size() * sizeof(F)) == 0;
		std::cerr << (errors == 0 ? "OK" : "FAILED") << " (centroid error relative to rms coordinate: " << centroidErr
			<< (identical ? "; bit-identical to the serial run" : "") << ")" << std::endl;
	}

	if (args.isPresent("dump")) {
		dumpVector(args.getString("dump") + (sizeof(F) == 8 ? ".means.f64" : ".means.f32"), algorithm->getMeans());
		dumpVector(args.getString("dump") + ".assignment.u32", algorithm->getAssignment());
	}

	if (json) {
		auto* hip = dynamic_cast<HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, Best, Shm>*>(algorithm.get());
		auto* ordered = dynamic_cast<HipKMeansAlgorithm<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC, Best, Ordered>*>(algorithm.get());
		std::cout << "{\"algorithm\": \"" << algoName << "\", \"n\": " << n << ", \"dim\": " << dim << ", \"k\": " << k
			<< ", \"iterations\": " << iters << ", \"init_ms\": " << initMs << ", \"ms_per_iteration\": " << msPerIter
			<< ", \"ns_per_input_float\": " << nsPerFloat
			<< ", \"points_centroids_dims_per_s\": " << (double)n * (double)k * (double)dim / (msPerIter * 1e-3);
		if (hip) std::cout << ", \"assign_ms\": " << hip->assignMs() / (double)iters << ", \"update_ms\": " << hip->updateMs() / (double)iters
			<< ", \"rechecked_points\": " << hip->recheckedPoints();
		if (ordered) std::cout << ", \"assign_ms\": " << ordered->assignMs() / (double)iters << ", \"update_ms\": " << ordered->updateMs() / (double)iters
			<< ", \"rechecked_points\": " << ordered->recheckedPoints();
		if (verified) std::cout << ", \"verify_errors\": " << errors << ", \"assignment_mismatches\": " << mismatches
			<< ", \"centroid_error\": " << centroidErr << ", \"bit_identical\": " << (identical ? "true" : "false");
		std::cout << "}" << std::endl;
	}
	algorithm->cleanup();
}

template<typename F, class LAYOUT, class LAYOUT_MEANS>
void run(const ProgramArguments& args)
{
	using METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT_MEANS>;
	const std::size_t dim = (std::size_t)args.getInt("dim"), k = (std::size_t)args.getInt("k"), n = (std::size_t)args.getInt("N");
	const std::size_t seed = (std::size_t)args.getInt("seed");
	if (k > n) throw std::runtime_error("k must not exceed N.");

	std::cerr << "Generating input data (" << n << " x " << dim << ") ..." << std::endl;
	if (args.isPresent("seed")) std::cerr << "Seed is set to " << seed << std::endl;
	std::vector<F> data, means;
	const std::string dataset = args.getString("dataset");
	if (dataset == "benchmark") {
		kmx_dataset_spec spec;
		if (kmx_gen_baseline_config((int)args.getInt("config"), &spec) != 0) throw std::runtime_error("Unknown benchmark configuration.");
		if (spec.dim != dim || spec.k != k) throw std::runtime_error("internal: benchmark configuration and arguments disagree");
		generate_benchmark_data<F, LAYOUT>(data, spec, n);
	}
	else generate_clustered_data<F, LAYOUT>(data, n, k, dim, seed);

	if (args.getString("init") == "first") first_k_means<F, LAYOUT, LAYOUT_MEANS>(data, means, n, k, dim);
	else prepare_means<F, std::uint32_t, LAYOUT, LAYOUT_MEANS>(data, means, n, k, dim, true, seed);

	if (args.getBool("assignmentOnly")) run_assignment<F, std::uint32_t, LAYOUT, LAYOUT_MEANS, METRIC>(args, data, means);
	else run_kmeans<F, std::uint32_t, LAYOUT, LAYOUT_MEANS, METRIC>(args, data, means);
	std::cerr << "And we're done here." << std::endl;
}

template<typename F, class LAYOUT>
void select_layout2_and_run(const ProgramArguments& args)
{
	if (!args.isPresent("layoutMeans")) { run<F, LAYOUT, LAYOUT>(args); return; }
	const std::string layout = args.getString("layoutMeans");
	if (layout == "soa") run<F, LAYOUT, SoALayoutPolicy<1>>(args);
	else if (layout == "aos") run<F, LAYOUT, AoSLayoutPolicy<1>>(args);
	else throw std::runtime_error("Unknown data layout '" + layout + "'.");
}

template<typename F>
void select_layout_and_run(const ProgramArguments& args)
{
	const std::string layout = args.getString("layout");
	if (layout == "soa") select_layout2_and_run<F, SoALayoutPolicy<1>>(args);
	else if (layout == "aos") select_layout2_and_run<F, AoSLayoutPolicy<1>>(args);
	else throw std::runtime_error("Unknown data layout '" + layout + "'.");
}

} // namespace

int main(int argc, char* argv[])
{
	ProgramArguments args;
	try {
		args.registerInt("dim", "Vector dimension.", 20, 2);
		args.registerInt("k", "Number of buckets.", 128, 2);
		args.registerInt("N", "Number of vectors in a batch.", 10240, 128);
		args.registerInt("iterations", "Iterations to be performed.", 1, 1);
		args.registerInt("seed", "Random generator seed.", 42, 0);
		args.registerBool("assignmentOnly", "Run only assignment part of the algorithm (microbenchmark).");
		args.conflicts("assignmentOnly", "iterations");
		args.registerString("algorithm", "Which algorithm is to be tested (serial, hip_base, hip_base_shm, hip_mfma, hip_mfma_bf16, hip_best, hip_best_serial_order, hip_fused; assignment only: hip_lds_fma).", "serial");
		args.registerEnum("layout", "Type of data layout.", "aos", { "aos", "soa" });
		args.registerEnum("layoutMeans", "Type of data layout (override for means only).", "aos", { "aos", "soa" });
		args.registerBool("double", "Use doubles instead of floats.");
		args.registerBool("verify", "Verify results against base (serial) algorithm.");
		args.registerInt("privatizedCopies", "Number of privatized copies in global memory (relevant only to some algorithms).", 1, 1, 4096);
		args.registerInt("itemsPerThread", "Number of computations performed per thread.", 1, 1, 4096);
		args.registerInt("regsCache", "Size of the registry cache (accepted for compatibility; no kernel of this build reads it, a warning says so).", 1, 1);
		args.registerInt("cudaBlockSize", "Number of threads in each block.", 256, 1, 4096);
		args.alias("hipBlockSize", "cudaBlockSize");
		args.registerInt("cudaBlockCount", "Number of blocks executed in a grid (algorithms choose their own).", 0, 0);
		args.alias("hipBlockCount", "cudaBlockCount");
		args.registerInt("cudaSharedMemorySize", "Amount of LDS allowed per block (0 = device maximum).", 0, 0);
		args.alias("hipSharedMemorySize", "cudaSharedMemorySize");
		/* additions */
		args.registerEnum("dataset", "reference = the reference's generator; benchmark = seeded benchmark configuration (--config).", "reference", { "reference", "benchmark" });
		args.registerInt("config", "Benchmark configuration 1..5 (sets dim, k, N, iterations unless given; implies --dataset benchmark --init first).", 0, 0, 5);
		args.registerEnum("init", "Initial centroids: k shuffled points (reference) or the first k points.", "shuffle", { "shuffle", "first" });
		args.registerInt("serialThreads", "Threads of the serial algorithm (results are bit-identical to 1 thread).", 1, 1, 1024);
		args.registerBool("json", "Print a JSON report instead of the two-number line.");
		args.registerBool("graph", "Record a pair of iterations as a HIP graph and replay it instead of launching every kernel (device algorithms; not with --json).");
		args.registerString("dump", "Write the final centroids and assignment to <prefix>.means.f32 (.f64 with --double) / <prefix>.assignment.u32.", "");
		args.process(argc, argv);
	}
	catch (ArgumentException& e) {
		std::cout << "Invalid arguments: " << e.what() << std::endl << std::endl;
		args.printUsage(std::cout);
		return 1;
	}

	try {
		const bool useDouble = args.getBool("double");
		if (args.getInt("config") > 0) {
			/* a benchmark configuration fixes the shape; explicit arguments may shrink N or the iteration count */
			kmx_dataset_spec spec;
			kmx_gen_baseline_config((int)args.getInt("config"), &spec);
			std::vector<std::string> forced = { "k-means", "--dataset", "benchmark", "--init", "first",
				"--dim", std::to_string(spec.dim), "--k", std::to_string(spec.k) };
			if (!args.isPresent("N")) { forced.push_back("--N"); forced.push_back(std::to_string(spec.n)); }
			if (!args.isPresent("iterations") && !args.getBool("assignmentOnly")) { forced.push_back("--iterations"); forced.push_back(std::to_string(spec.iterations)); }
			std::vector<char*> argv2;
			for (int i = 0; i < argc; ++i) argv2.push_back(argv[i]);
			for (std::size_t i = 1; i < forced.size(); ++i) argv2.push_back(const_cast<char*>(forced[i].c_str()));
			ProgramArguments again = args; /* same registrations, re-parse with the forced values appended */
			again.process((int)argv2.size(), argv2.data());
			if (useDouble) select_layout_and_run<double>(again);
			else select_layout_and_run<float>(again);
		}
		else if (useDouble) select_layout_and_run<double>(args);
		else select_layout_and_run<float>(args);
	}
	catch (ArgumentException& e) {
		std::cout << "Invalid arguments: " << e.what() << std::endl << std::endl;
		return 1;
	}
	catch (std::exception& e) {
		std::cout << "Error: " << e.what() << std::endl << std::endl;
		return 2;
	}
	return 0;
}
