/*
 * train_steps.cpp — whole training steps on the device from C++, through cattle_hip/DeviceNet.hpp: the two
 * feed-forward configurations of the benchmark definition and the network of the reference's own example
 * (examples/cifar_convnet.cpp:24-41), built layer by layer as a C-ATTL3 user would build them, trained with
 * DeviceFeedforwardNetwork::train_batch* (one batch of SGDOptimizer::_train, optimizer/SGDOptimizer.hpp:44-70:
 * propagate, loss, gradient / batch size, backpropagate, update, reset) on synthetic data, and timed. Prints one
 * JSON line.
 *
 *   g++ -std=c++11 -O2 -I include -I c-attl3_amd/include c-attl3_amd/examples/train_steps.cpp \
 *       -L c-attl3_amd -lcattle_hip -Wl,-rpath,'$ORIGIN/..' -o c-attl3_amd/examples/train_steps
 *   c-attl3_amd/examples/train_steps [steps] [warmup]
 */
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "cattle_hip/DeviceNet.hpp"

using namespace cattle::hip::device;

typedef float Scalar;
typedef DeviceTensor<Scalar> DT;
typedef DeviceLayer<Scalar> DL;
typedef DL::Dims Dims;

struct Lcg {
	std::uint64_t s;
	explicit Lcg(std::uint64_t seed) : s(seed * 2862933555777941757ULL + 3037000493ULL) { }
	double next() {                 /* uniform in [-1, 1) */
		s = s * 6364136223846793005ULL + 1442695040888963407ULL;
		return (double) (s >> 11) / 9007199254740992.0 * 2.0 - 1.0;
	}
};

static std::vector<Scalar> random_values(std::size_t count, Lcg& g, double scale) {
	std::vector<Scalar> v(count);
	for (std::size_t i = 0; i < count; ++i)
		v[i] = (Scalar) (g.next() * scale);
	return v;
}

/* weight matrices uniform with the variance of He initialisation (2 / fan_in); biases, gamma, beta keep their initial values */
static void init_weights(DeviceFeedforwardNetwork<Scalar>& net, Lcg& g) {
	std::vector<DL>& layers = net.get_layers();
	for (std::size_t l = 0; l < layers.size(); ++l)
		for (std::size_t p = 0; p < layers[l].num_params(); ++p) {
			std::size_t rows, cols;
			bool optimizable;
			layers[l].param_shape(p, rows, cols, optimizable);
			if (optimizable && rows > 1) {
				std::vector<Scalar> w = random_values(rows * cols, g, std::sqrt(6.0 / (double) rows));
				layers[l].set_param_values(p, w.data());
			}
		}
}

static std::vector<Scalar> one_hot(std::size_t batch, std::size_t classes, Lcg& g) {
	std::vector<Scalar> y(batch * classes, (Scalar) 0);
	for (std::size_t n = 0; n < batch; ++n) {
		std::size_t c = (std::size_t) ((g.next() + 1.0) / 2.0 * (double) classes);
		y[n + batch * (c < classes ? c : classes - 1)] = 1;
	}
	return y;
}

template<typename Step>
static double time_steps(std::size_t steps, std::size_t warmup, Step step) {
	for (std::size_t t = 0; t < warmup; ++t)
		step(t);
	check(cattle_hip_synchronize());
	const std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
	for (std::size_t t = 0; t < steps; ++t)
		step(warmup + t);
	check(cattle_hip_synchronize());
	return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / (double) steps;
}

int main(int argc, char** argv) {
	const std::size_t steps = argc > 1 ? (std::size_t) std::atol(argv[1]) : 50;
	const std::size_t warmup = argc > 2 ? (std::size_t) std::atol(argv[2]) : 5;
	try {
		check(cattle_hip_init(0));
		DeviceLoss<Scalar> loss(CATTLE_HIP_LOSS_SOFTMAX_CROSS_ENTROPY);
		Lcg g(2);
		double mlp_ms, conv_ms, cifar_ms, mlp_fused_ms, conv_fused_ms, cifar_fused_ms, mlp_rec_ms, conv_rec_ms;
		{
			/* MLP 784-512-256-10 with ReLU, batch 256, vanilla SGD */
			const std::size_t batch = 256;
			std::vector<DL> layers;
			layers.push_back(DL::dense(Dims{ { 784, 1, 1 } }, 512));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
			layers.push_back(DL::dense(layers.back().get_output_dims(), 256));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
			layers.push_back(DL::dense(layers.back().get_output_dims(), 10));
			DeviceFeedforwardNetwork<Scalar> net(std::move(layers));
			init_weights(net, g);
			std::vector<Scalar> x = random_values(batch * 784, g, 1.0), y = one_hot(batch, 10, g);
			DT xd(DT::Dims{ { batch, 784, 1, 1 } }, x.data()), yd(DT::Dims{ { batch, 10, 1, 1 } }, y.data());
			mlp_ms = time_steps(steps, warmup, [&](std::size_t) { net.train_batch_sgd(xd, yd, loss, (Scalar) 1e-3); });
			/* the same network with each dense layer and its ReLU run as one fused layer */
			net.fuse();
			mlp_fused_ms = time_steps(steps, warmup, [&](std::size_t) { net.train_batch_sgd(xd, yd, loss, (Scalar) 1e-3); });
			/* the fused step recorded once and launched as a graph: one call instead of fourteen before the loss is read back */
			DeviceFeedforwardNetwork<Scalar>::RecordedBatch rec = net.record_batch(xd, yd, loss);
			const double sgd[4] = { 1e-3, 0, 0, 0 };
			mlp_rec_ms = time_steps(steps, warmup, [&](std::size_t) { rec.run(CATTLE_HIP_OPT_VANILLA_SGD, sgd, 0, 0); });
		}
		{
			/* conv 3x3x32 - ReLU - max pool - conv 3x3x64 - batch norm - ReLU - max pool - dense 10, batch 128, Adam */
			const std::size_t batch = 128;
			std::vector<DL> layers;
			layers.push_back(DL::conv(Dims{ { 32, 32, 3 } }, 32));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
			layers.push_back(DL::pool(CATTLE_HIP_POOL_MAX, layers.back().get_output_dims()));
			layers.push_back(DL::conv(layers.back().get_output_dims(), 64));
			layers.push_back(DL::batch_norm(layers.back().get_output_dims()));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
			layers.push_back(DL::pool(CATTLE_HIP_POOL_MAX, layers.back().get_output_dims()));
			layers.push_back(DL::dense(layers.back().get_output_dims(), 10));
			DeviceFeedforwardNetwork<Scalar> net(std::move(layers));
			init_weights(net, g);
			std::vector<Scalar> x = random_values(batch * 32 * 32 * 3, g, 1.0), y = one_hot(batch, 10, g);
			DT xd(DT::Dims{ { batch, 32, 32, 3 } }, x.data()), yd(DT::Dims{ { batch, 10, 1, 1 } }, y.data());
			conv_ms = time_steps(steps, warmup, [&](std::size_t t) { net.train_batch_adam(xd, yd, loss, t); });
			/* conv-ReLU-pool and conv-BN-ReLU-pool as fused layers */
			net.fuse();
			conv_fused_ms = time_steps(steps, warmup, [&](std::size_t t) { net.train_batch_adam(xd, yd, loss, steps + warmup + t); });
			DeviceFeedforwardNetwork<Scalar>::RecordedBatch rec = net.record_batch(xd, yd, loss);
			const double adam[4] = { 1e-3, 1e-1, 1e-3, 1e-5 };
			conv_rec_ms = time_steps(steps, warmup, [&](std::size_t t) { rec.run(CATTLE_HIP_OPT_ADAM, adam, 0, 2 * (steps + warmup) + t); });
		}
		{
			/* examples/cifar_convnet.cpp:24-41: conv 3x3x8 - ReLU - max pool - conv 3x3x8 - ReLU - max pool - dropout .25 -
			 * dense 50 - ReLU - dropout .5 - dense 10 - softmax; CrossEntropyLoss; NadamOptimizer, batch 200 */
			const std::size_t batch = 200;
			std::vector<DL> layers;
			layers.push_back(DL::conv(Dims{ { 32, 32, 3 } }, 8));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
			layers.push_back(DL::pool(CATTLE_HIP_POOL_MAX, layers.back().get_output_dims()));
			layers.push_back(DL::conv(layers.back().get_output_dims(), 8));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
			layers.push_back(DL::pool(CATTLE_HIP_POOL_MAX, layers.back().get_output_dims()));
			layers.push_back(DL::dropout(layers.back().get_output_dims(), (Scalar) .25, 1));
			layers.push_back(DL::dense(layers.back().get_output_dims(), 50));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
			layers.push_back(DL::dropout(layers.back().get_output_dims(), (Scalar) .5, 2));
			layers.push_back(DL::dense(layers.back().get_output_dims(), 10));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_SOFTMAX, layers.back().get_output_dims(), (Scalar) 1e-5));
			DeviceFeedforwardNetwork<Scalar> net(std::move(layers));
			/* the example's initializations (examples/cifar_convnet.cpp:21-22): He for the convolutions, Glorot for the
			 * dense layers, both scaled by 0.1 */
			const HeParameterInitialization<Scalar> conv_init((Scalar) 1e-1);
			const GlorotParameterInitialization<Scalar> dense_init((Scalar) 1e-1);
			net.get_layers()[0].init_params(0, conv_init);
			net.get_layers()[3].init_params(0, conv_init);
			net.get_layers()[7].init_params(0, dense_init);
			net.get_layers()[10].init_params(0, dense_init);
			std::vector<Scalar> x = random_values(batch * 32 * 32 * 3, g, 0.5), y = one_hot(batch, 10, g);
			for (std::size_t i = 0; i < x.size(); ++i)
				x[i] += (Scalar) 0.5;                                   /* pixel values in [0, 1) */
			DT xd(DT::Dims{ { batch, 32, 32, 3 } }, x.data()), yd(DT::Dims{ { batch, 10, 1, 1 } }, y.data());
			DeviceLoss<Scalar> cross_entropy(CATTLE_HIP_LOSS_CROSS_ENTROPY);
			const double nadam[4] = { 1e-3, 1e-1, 1e-3, 1e-5 };        /* optimizer/NadamOptimizer.hpp:39-41 */
			cifar_ms = time_steps(steps, warmup, [&](std::size_t t) {
				net.train_batch(xd, yd, cross_entropy, CATTLE_HIP_OPT_NADAM, nadam, 0, t);
			});
			net.fuse();
			cifar_fused_ms = time_steps(steps, warmup, [&](std::size_t t) {
				net.train_batch(xd, yd, cross_entropy, CATTLE_HIP_OPT_NADAM, nadam, 0, steps + warmup + t);
			});
		}
		std::printf("{\"driver\": \"C++ (cattle_hip/DeviceNet.hpp), train_batch* incl. the per-batch loss read-back\", "
				"\"steps\": %zu, \"warmup\": %zu, \"mlp_784_512_256_10_batch256_sgd_ms\": %.4f, \"convnet_32x32x3_batch128_adam_ms\": %.4f, "
				"\"reference_cifar_example_batch200_nadam_ms\": %.4f, \"fused\": {\"mlp_784_512_256_10_batch256_sgd_ms\": %.4f, "
				"\"convnet_32x32x3_batch128_adam_ms\": %.4f, \"reference_cifar_example_batch200_nadam_ms\": %.4f}, "
				"\"fused_and_recorded_as_hip_graph\": {\"mlp_784_512_256_10_batch256_sgd_ms\": %.4f, \"convnet_32x32x3_batch128_adam_ms\": %.4f}}\n",
				steps, warmup, mlp_ms, conv_ms, cifar_ms, mlp_fused_ms, conv_fused_ms, cifar_fused_ms, mlp_rec_ms, conv_rec_ms);
	} catch (const std::exception& e) {
		std::fprintf(stderr, "train_steps: %s\n", e.what());
		return 1;
	}
	return 0;
}
