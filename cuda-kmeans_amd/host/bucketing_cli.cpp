/*
 * Command-line harness of the update micro-benchmark: sums N random vectors into k buckets, one independent batch
 * per iteration, and prints "<ms per batch> <ns per input float>" like the reference's bucketing-cuda
 * (experimental/bucketing-cuda/bucketing-cuda/bucketing-cuda.cpp:161-218; options :243-272; verification with a
 * relative tolerance of 5e-5 :104-142). Inputs: data uniform in [0,1), indices uniform in [0,k), from mt19937(seed)
 * as in the reference (:177-178).
 *
 * Algorithms: serial, hip_base, hip_atomic_point, hip_atomic_warp, hip_atomic_fine, hip_atomic_shm, hip_atomic_shm2,
 * hip_fake, hip_fake_shm (the reference's cuda_* names are accepted), --emul. The two "fake" algorithms are probes of the
 * raw cost of atomic additions (bucketing-cuda/kernels/kernels.cu:452-531): they ignore the inputs and add the constant
 * 0.1 to bucket (i / dim) % k, so --verify checks them against that closed form instead of the serial sums.
 * --double: the serial algorithm and the atomic point, fine and shm kernels.
 */
#include "bucketing.hpp"
#include "cli_args.hpp"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <fstream>
#include <iostream>
#include <limits>
#include <map>
#include <memory>
#include <random>
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

template<typename T, class DIST>
void generate_random(std::vector<T>& data, DIST distribution, std::size_t seed)
{
	std::mt19937 generator((unsigned int)seed);
	for (auto& x : data) x = distribution(generator);
}

std::string canonicalAlgorithm(const std::string& name)
{
	static const std::map<std::string, std::string> aliases = {
		{ "cuda_base", "hip_base" }, { "cuda_atomic_point", "hip_atomic_point" }, { "cuda_atomic_warp", "hip_atomic_warp" },
		{ "cuda_atomic_fine", "hip_atomic_fine" }, { "cuda_atomic_shm", "hip_atomic_shm" }, { "cuda_atomic_shm2", "hip_atomic_shm2" },
		{ "cuda_fake", "hip_fake" }, { "cuda_fake_shm", "hip_fake_shm" },
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
}

/* relative error |a-b| / max(|a|+|b|, tol) above tol counts as an error (bucketing-cuda.cpp:104-142) */
template<typename F>
bool verify(const std::vector<F>& res, const std::vector<F>& correctRes, std::size_t dims, std::size_t k)
{
	if (res.size() != correctRes.size()) {
		std::cerr << std::endl << "Error: Result size mismatch (" << res.size() << " values found, but " << correctRes.size() << " values expected)!" << std::endl;
		return false;
	}
	constexpr double tolerance = 0.00005;
	std::size_t errors = 0;
	for (std::size_t i = 0; i < res.size(); ++i) {
		const double a = (double)res[i], b = (double)correctRes[i];
		const double err = std::abs(a - b) / std::max(std::abs(a) + std::abs(b), tolerance);
		if (!(err <= tolerance)) {
			if (errors == 0) std::cerr << std::endl;
			if (++errors <= 10)
				std::cerr << "Error at iteration #" << (i / dims) / k << " [" << (i / dims) % k << "][" << (i % dims) << "]: "
					<< res[i] << " != " << correctRes[i] << std::endl;
		}
	}
	if (errors > 0) std::cerr << "Total errors found: " << errors << std::endl;
	return errors == 0;
}

template<typename F>
void saveResults(const std::string& fileName, const std::vector<F>& result, std::size_t dim)
{
	std::ofstream out(fileName);
	if (!out) throw std::runtime_error("Cannot open '" + fileName + "' for writing.");
	for (std::size_t i = 0; i < result.size(); ++i)
		out << result[i] << ((i + 1) % dim == 0 ? '\n' : ' ');
}

template<typename F, class LAYOUT>
void run(const ProgramArguments& args)
{
	const std::size_t dim = (std::size_t)args.getInt("dim"), k = (std::size_t)args.getInt("k"), n = (std::size_t)args.getInt("N");
	const std::size_t iter = (std::size_t)args.getInt("iterations");
	const std::size_t seed = (std::size_t)args.getInt("seed");

	std::vector<F> data(LAYOUT::size(n, dim) * iter);
	std::vector<std::uint32_t> indices(n * iter);
	std::cerr << "Generating input data (" << n << " x " << dim << "), " << iter << " iterations ..." << std::endl;
	if (args.isPresent("seed")) std::cerr << "Seed is set to " << seed << std::endl;
	generate_random(data, std::uniform_real_distribution<F>((F)0.0, (F)1.0), seed);
	generate_random(indices, std::uniform_int_distribution<std::uint32_t>(0, (std::uint32_t)k - 1), seed);

	const std::string algoName = canonicalAlgorithm(args.getString("algorithm"));
	const bool fake = algoName == "hip_fake" || algoName == "hip_fake_shm";
	HipExecParameters exec;
	getHipExecParameters(args, exec);
	std::map<std::string, std::unique_ptr<IBucketingAlgorithm<F>>> algorithms;
	algorithms["serial"].reset(new SerialBucketingAlgorithm<F, LAYOUT>());
	algorithms["hip_base"].reset(new HipBucketingAlgorithm<F, LAYOUT, BaseKernel<F, LAYOUT>>(exec));
	if (args.getBool("emul")) {
		algorithms["hip_atomic_point"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicPointKernel<F, LAYOUT, true>>(exec));
		algorithms["hip_atomic_warp"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicWarpKernel<F, LAYOUT, true>>(exec));
		algorithms["hip_atomic_fine"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicFineKernel<F, LAYOUT, true>>(exec));
		algorithms["hip_atomic_shm"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicShmKernel<F, LAYOUT, true>>(exec));
		algorithms["hip_fake"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicFakeKernel<F, LAYOUT, true>>(exec));
	}
	else {
		algorithms["hip_atomic_point"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicPointKernel<F, LAYOUT>>(exec));
		algorithms["hip_atomic_warp"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicWarpKernel<F, LAYOUT>>(exec));
		algorithms["hip_atomic_fine"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicFineKernel<F, LAYOUT>>(exec));
		algorithms["hip_atomic_shm"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicShmKernel<F, LAYOUT>>(exec));
		algorithms["hip_fake"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicFakeKernel<F, LAYOUT>>(exec));
	}
	algorithms["hip_atomic_shm2"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicShm2Kernel<F, LAYOUT>>(exec));
	algorithms["hip_fake_shm"].reset(new HipBucketingAlgorithm<F, LAYOUT, AtomicShmFakeKernel<F, LAYOUT>>(exec));
	auto it = algorithms.find(algoName);
	if (it == algorithms.end()) throw std::runtime_error("Unkown algorithm '" + algoName + "'.");
	std::cerr << "Selected algorithm: " << algoName << std::endl;
	auto algorithm = std::move(it->second);

	Stopwatch stopwatch;
	std::cerr << "Initializing ... "; std::cerr.flush();
	stopwatch.start();
	algorithm->initialize(dim, k, n, iter, data, indices);
	stopwatch.stop();
	std::cerr << stopwatch.getMiliseconds() << " ms" << std::endl;

	std::cerr << "Running ... "; std::cerr.flush();
	stopwatch.start();
	algorithm->run();
	stopwatch.stop();
	std::cout << (stopwatch.getMiliseconds() / (double)iter); std::cout.flush();
	std::cerr << " ms/iter (which is"; std::cerr.flush();
	std::cout << " " << (stopwatch.getMiliseconds() * 1000000.0 / (double)(iter * dim * n)); std::cout.flush();
	std::cerr << " ns/input float)"; std::cerr.flush();
	std::cout << std::endl;

	if (args.getBool("verify")) {
		std::cerr << "Verifying results ... "; std::cerr.flush();
		if (fake) {
			/* what the probes add up to: 0.1 per point whose number is congruent to the bucket modulo k, in every dimension */
			std::vector<F> expected(iter * k * dim); /* getResult() is iterations x k rows of dim sums, whatever the layout */
			for (std::size_t i = 0; i < expected.size(); ++i) {
				const std::size_t b = (i / dim) % k;
				expected[i] = (F)(0.1 * (double)(n / k + (b < n % k ? 1 : 0)));
			}
			std::cerr << (verify(algorithm->getResult(), expected, dim, k) ? "OK" : "FAILED") << std::endl;
		}
		else {
			SerialBucketingAlgorithm<F, LAYOUT> base;
			base.initialize(dim, k, n, iter, data, indices);
			base.run();
			std::cerr << (verify(algorithm->getResult(), base.getResult(), dim, k) ? "OK" : "FAILED") << std::endl;
		}
	}
	if (args.isPresent("out")) {
		std::cerr << "Saving results to " << args.getString("out") << " ..." << std::endl;
		saveResults(args.getString("out"), algorithm->getResult(), dim);
	}
	algorithm->cleanup();
	std::cerr << "And we're done here." << std::endl;
}

template<typename F>
void select_layout_and_run(const ProgramArguments& args)
{
	const std::string layout = args.getString("layout");
	if (layout == "soa") run<F, SoALayoutPolicy<1>>(args);
	else if (layout == "soa32") run<F, SoALayoutPolicy<32>>(args);
	else if (layout == "aos") run<F, AoSLayoutPolicy<1>>(args);
	else if (layout == "aos32") run<F, AoSLayoutPolicy<32>>(args);
	else throw std::runtime_error("Unknown data layout '" + layout + "'.");
}

} // namespace

int main(int argc, char* argv[])
{
	ProgramArguments args;
	try {
		args.registerInt("dim", "Vector dimension.", 20, 2);
		args.registerInt("k", "Number of buckets.", 512, 2);
		args.registerInt("N", "Number of vectors in a batch.", 10240, 128);
		args.registerInt("iterations", "Iterations to be performed (i.e., number of batches).", 1, 1);
		args.registerInt("seed", "Random generator seed.", 42, 0);
		args.registerString("algorithm", "Which algorithm is to be tested (serial, hip_base, hip_atomic_point, hip_atomic_warp, hip_atomic_fine, hip_atomic_shm, hip_atomic_shm2, hip_fake, hip_fake_shm).", "serial");
		args.registerBool("emul", "Emulate atomic additions with atomic CAS operations (point, warp, fine and fake algorithms).");
		args.registerEnum("layout", "Type of data layout and alignment.", "aos", { "aos", "soa", "aos32", "soa32" });
		args.registerBool("double", "Use doubles instead of floats (serial, hip_atomic_point, hip_atomic_fine, hip_atomic_shm).");
		args.registerBool("verify", "Verify results against base (serial) algorithm.");
		args.registerString("out", "Path to a file where the results are saved.", "");
		args.registerInt("privatizedCopies", "Number of privatized copies in global memory (relevant only to some algorithms).", 1, 1, 4096);
		args.registerInt("itemsPerThread", "Number of computations performed per thread.", 1, 1);
		args.registerInt("cudaBlockSize", "Number of threads in each block.", 256, 1, 4096);
		args.alias("hipBlockSize", "cudaBlockSize");
		args.registerInt("cudaBlockCount", "Number of blocks executed in a grid (algorithms choose their own).", 0, 0);
		args.alias("hipBlockCount", "cudaBlockCount");
		args.registerInt("cudaSharedMemorySize", "Amount of LDS allowed per block (0 = device maximum).", 0, 0);
		args.alias("hipSharedMemorySize", "cudaSharedMemorySize");
		args.process(argc, argv);
	}
	catch (ArgumentException& e) {
		std::cout << "Invalid arguments: " << e.what() << std::endl << std::endl;
		args.printUsage(std::cout);
		return 1;
	}

	try {
		if (args.getBool("double")) select_layout_and_run<double>(args);
		else select_layout_and_run<float>(args);
	}
	catch (std::exception& e) {
		std::cout << "Error: " << e.what() << std::endl << std::endl;
		return 2;
	}
	return 0;
}
