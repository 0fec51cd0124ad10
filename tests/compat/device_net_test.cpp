/*
 * device_net_test.cpp — drives cattle_hip/DeviceNet.hpp (device tensors chained between layers, loss and
 * optimizer update on the device) through three training batches of two small networks and records the
 * inputs, the initial parameters, the batch losses and the final parameters to a file that
 * tests/test_gpu_device_net.py replays on the CPU oracle.
 *
 *   mlp:     dense 20 -> 16, ReLU, dense 16 -> 6, softmax cross-entropy, vanilla SGD
 *   convnet: conv 8x8x3 -> 8 filters 3x3 p1, ReLU, max pool 2x2, batch norm, dense -> 5, softmax
 *            cross-entropy, Adam
 */
#include "cattle_hip/DeviceNet.hpp"

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <random>
#include <string>

using namespace cattle::hip::device;

static FILE* g_out = nullptr;

static void record(const std::string& name, std::size_t scalar_size, const std::vector<std::size_t>& dims, const void* data) {
	std::uint32_t len = (std::uint32_t) name.size(), ss = (std::uint32_t) scalar_size, rank = (std::uint32_t) dims.size();
	std::fwrite(&len, 4, 1, g_out);
	std::fwrite(name.data(), 1, len, g_out);
	std::fwrite(&ss, 4, 1, g_out);
	std::fwrite(&rank, 4, 1, g_out);
	std::size_t count = 1;
	for (std::size_t d : dims) {
		std::uint64_t v = d;
		std::fwrite(&v, 8, 1, g_out);
		count *= d;
	}
	std::fwrite(data, scalar_size, count, g_out);
}

/* deterministic inputs: a 64-bit LCG mapped to [-1, 1) */
struct Lcg {
	std::uint64_t s;
	explicit Lcg(std::uint64_t seed) : s(seed * 2862933555777941757ULL + 3037000493ULL) { }
	double next() {
		s = s * 6364136223846793005ULL + 1442695040888963407ULL;
		return (double) (s >> 11) / 9007199254740992.0 * 2.0 - 1.0;
	}
};

template<typename Scalar>
static std::vector<Scalar> random_values(std::size_t count, Lcg& g, double scale) {
	std::vector<Scalar> v(count);
	for (std::size_t i = 0; i < count; ++i)
		v[i] = (Scalar) (g.next() * scale);
	return v;
}

template<typename Scalar>
static void init_and_record(const std::string& tag, DeviceFeedforwardNetwork<Scalar>& net, Lcg& g) {
	std::vector<DeviceLayer<Scalar>>& layers = net.get_layers();
	for (std::size_t l = 0; l < layers.size(); ++l)
		for (std::size_t p = 0; p < layers[l].num_params(); ++p) {
			std::size_t rows, cols;
			bool opt;
			layers[l].param_shape(p, rows, cols, opt);
			if (opt && rows > 1) {      /* weight matrices; biases, gamma, beta keep their initial values */
				std::vector<Scalar> w = random_values<Scalar>(rows * cols, g, std::sqrt(6.0 / (double) rows));
				layers[l].set_param_values(p, w.data());
			}
			record(tag + ".init." + std::to_string(l) + "." + std::to_string(p), sizeof(Scalar), { rows, cols },
					layers[l].get_param_values(p).data());
		}
}

template<typename Scalar>
static void record_final(const std::string& tag, DeviceFeedforwardNetwork<Scalar>& net) {
	std::vector<DeviceLayer<Scalar>>& layers = net.get_layers();
	for (std::size_t l = 0; l < layers.size(); ++l)
		for (std::size_t p = 0; p < layers[l].num_params(); ++p) {
			std::size_t rows, cols;
			bool opt;
			layers[l].param_shape(p, rows, cols, opt);
			record(tag + ".final." + std::to_string(l) + "." + std::to_string(p), sizeof(Scalar), { rows, cols },
					layers[l].get_param_values(p).data());
			/* every step ends with reset_grad (optimizer/SGDOptimizer.hpp:68-70) */
			std::vector<Scalar> grad = layers[l].get_param_grad(p);
			for (Scalar v : grad)
				if (v != 0)
					throw std::runtime_error("gradient not reset after the step");
		}
}

template<typename Scalar>
static std::vector<Scalar> one_hot(std::size_t batch, std::size_t classes, Lcg& g) {
	std::vector<Scalar> y(batch * classes, (Scalar) 0);
	for (std::size_t n = 0; n < batch; ++n) {
		std::size_t c = (std::size_t) ((g.next() + 1.0) / 2.0 * (double) classes);
		y[n + batch * (c < classes ? c : classes - 1)] = 1;
	}
	return y;
}

static std::string g_dir;      /* scratch directory for parameter files */

template<typename Scalar>
static void run(const std::string& tag) {
	typedef DeviceTensor<Scalar> DT;
	typedef DeviceLayer<Scalar> DL;
	typedef typename DL::Dims Dims;
	const std::size_t steps = 3;
	DeviceLoss<Scalar> loss(CATTLE_HIP_LOSS_SOFTMAX_CROSS_ENTROPY);
	/* each of the two trained networks once layer by layer and once with DeviceFeedforwardNetwork::fuse() (records "...f") */
	for (int fused = 0; fused < 3; ++fused) {        /* 2: fused, and all batches after the first recorded once and launched as a graph ("...g") */
		const std::string mlp = tag + (fused == 2 ? ".mlpg" : fused ? ".mlpf" : ".mlp");
		Lcg g(11);
		const std::size_t batch = 24;
		std::vector<DL> layers;
		layers.push_back(DL::dense(Dims{ { 20, 1, 1 } }, 16));
		layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
		layers.push_back(DL::dense(layers.back().get_output_dims(), 6));
		DeviceFeedforwardNetwork<Scalar> net(std::move(layers));
		if (fused) {
			const Scalar groups = (Scalar) net.fuse();
			record(mlp + ".groups", sizeof(Scalar), { 1 }, &groups);
		}
		init_and_record<Scalar>(mlp, net, g);
		std::vector<Scalar> x = random_values<Scalar>(batch * 20, g, 1.0), y = one_hot<Scalar>(batch, 6, g);
		record(mlp + ".x", sizeof(Scalar), { batch, 20 }, x.data());
		record(mlp + ".y", sizeof(Scalar), { batch, 6 }, y.data());
		DT xd(typename DT::Dims{ { batch, 20, 1, 1 } }, x.data()), yd(typename DT::Dims{ { batch, 6, 1, 1 } }, y.data());
		std::vector<Scalar> totals;
		if (fused == 2) {
			totals.push_back(net.train_batch_sgd(xd, yd, loss, (Scalar) 0.05));
			typename DeviceFeedforwardNetwork<Scalar>::RecordedBatch rec = net.record_batch(xd, yd, loss);
			const double sgd[4] = { (double) (Scalar) 0.05, 0, 0, 0 };
			for (std::size_t t = 1; t < steps; ++t)
				totals.push_back(rec.run(CATTLE_HIP_OPT_VANILLA_SGD, sgd, 0, 0));
		} else {
			for (std::size_t t = 0; t < steps; ++t)
				totals.push_back(net.train_batch_sgd(xd, yd, loss, (Scalar) 0.05));
		}
		record(mlp + ".losses", sizeof(Scalar), { steps }, totals.data());
		record_final<Scalar>(mlp, net);
	}
	{
		/* value and gradient constraints of a device-resident parameter (parameters/StandardParameters.hpp:105-123):
		 * values constrained when they are set, the gradient after the backward pass */
		Lcg g(15);
		const std::size_t batch = 6;
		DL dense = DL::dense(Dims{ { 7, 1, 1 } }, 4);
		dense.set_constraints(0, (Scalar) 0.3, (Scalar) 0.9, (Scalar) 0.5, (Scalar) 0.2, (Scalar) 0.6, (Scalar) 0.25);
		std::vector<Scalar> w = random_values<Scalar>(7 * 4, g, 1.0);
		dense.set_param_values(0, w.data());
		std::vector<Scalar> x = random_values<Scalar>(batch * 7, g, 1.0), go = random_values<Scalar>(batch * 4, g, 1.0);
		DT xd(typename DT::Dims{ { batch, 7, 1, 1 } }, x.data()), gd(typename DT::Dims{ { batch, 4, 1, 1 } }, go.data());
		dense.pass_forward_borrowed(xd, true);
		dense.pass_back(gd);
		record(tag + ".cons.w", sizeof(Scalar), { 7, 4 }, w.data());
		record(tag + ".cons.x", sizeof(Scalar), { batch, 7 }, x.data());
		record(tag + ".cons.go", sizeof(Scalar), { batch, 4 }, go.data());
		record(tag + ".cons.values", sizeof(Scalar), { 7, 4 }, dense.get_param_values(0).data());
		record(tag + ".cons.grad", sizeof(Scalar), { 7, 4 }, dense.get_param_grad(0).data());
	}
	{
		/* the data-movement layers of the reference's example networks: reshape -> broadcast -> dropout */
		Lcg g(14);
		const std::size_t batch = 5;
		std::vector<DL> layers;
		layers.push_back(DL::reshape(Dims{ { 12, 1, 1 } }, Dims{ { 3, 2, 2 } }));
		layers.push_back(DL::broadcast(layers.back().get_output_dims(), Dims{ { 2, 1, 3 } }));
		layers.push_back(DL::dropout(layers.back().get_output_dims(), (Scalar) 0.4, 321));
		DeviceFeedforwardNetwork<Scalar> net(std::move(layers), false);
		std::vector<Scalar> x = random_values<Scalar>(batch * 12, g, 1.0), go = random_values<Scalar>(batch * 72, g, 1.0);
		DT xd(typename DT::Dims{ { batch, 12, 1, 1 } }, x.data()), gd(typename DT::Dims{ { batch, 6, 2, 6 } }, go.data());
		record(tag + ".move.x", sizeof(Scalar), { batch, 12 }, x.data());
		record(tag + ".move.go", sizeof(Scalar), { batch, 6, 2, 6 }, go.data());
		record(tag + ".move.out", sizeof(Scalar), { batch, 6, 2, 6 }, net.propagate(xd, true).to_host().data());
		record(tag + ".move.dx", sizeof(Scalar), { batch, 12 }, net.backpropagate(gd).to_host().data());
		record(tag + ".move.infer", sizeof(Scalar), { batch, 6, 2, 6 }, net.propagate(xd, false).to_host().data());
	}
	{
		/* two stacked networks trained as the reference's generative-adversarial example trains them
		 * (examples/mnist_gan.cpp:92-109), once through DeviceStackedNetwork and the frozen flag, once with the same calls
		 * spelled out on two separate networks: the recorded parameters must be identical */
		const std::size_t batch = 12;
		const double adam[4] = { 2e-4, 0.5, 1e-3, 1e-5 };
		DeviceLoss<Scalar> bce(CATTLE_HIP_LOSS_BINARY_CROSS_ENTROPY);
		auto make_generator = [] {
			std::vector<DL> layers;
			layers.push_back(DL::dense(Dims{ { 1, 1, 10 } }, 24));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_LEAKY_RELU, layers.back().get_output_dims(), (Scalar) 0.2));
			layers.push_back(DL::dense(layers.back().get_output_dims(), 18));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_TANH, layers.back().get_output_dims()));
			layers.push_back(DL::reshape(layers.back().get_output_dims(), Dims{ { 3, 3, 2 } }));
			return DeviceFeedforwardNetwork<Scalar>(std::move(layers));
		};
		auto make_discriminator = [] {
			std::vector<DL> layers;
			layers.push_back(DL::dense(Dims{ { 3, 3, 2 } }, 16));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_LEAKY_RELU, layers.back().get_output_dims(), (Scalar) 0.2));
			layers.push_back(DL::dropout(layers.back().get_output_dims(), (Scalar) 0.3, 7));
			layers.push_back(DL::dense(layers.back().get_output_dims(), 1));
			layers.push_back(DL::activation(CATTLE_HIP_ACT_SIGMOID, layers.back().get_output_dims()));
			return DeviceFeedforwardNetwork<Scalar>(std::move(layers), false);
		};
		Lcg g(15);
		std::vector<Scalar> z = random_values<Scalar>(batch * 10, g, 1.0), real = random_values<Scalar>(batch * 18, g, 1.0);
		std::vector<Scalar> ones(batch, (Scalar) 1), zeros(batch, (Scalar) 0);
		DT zd(typename DT::Dims{ { batch, 1, 1, 10 } }, z.data()), reald(typename DT::Dims{ { batch, 3, 3, 2 } }, real.data());
		DT oned(typename DT::Dims{ { batch, 1, 1, 1 } }, ones.data()), zerod(typename DT::Dims{ { batch, 1, 1, 1 } }, zeros.data());
		for (int stacked = 0; stacked < 2; ++stacked) {
			Lcg gw(16);
			std::vector<DeviceFeedforwardNetwork<Scalar>> nets;
			nets.push_back(make_generator());
			nets.push_back(make_discriminator());
			init_and_record<Scalar>(tag + ".gan" + std::to_string(stacked) + ".g", nets[0], gw);
			init_and_record<Scalar>(tag + ".gan" + std::to_string(stacked) + ".d", nets[1], gw);
			std::vector<Scalar> losses;
			if (stacked) {
				DeviceStackedNetwork<Scalar> gan(std::move(nets));
				for (std::size_t t = 0; t < 2; ++t) {
					const DT& fake = gan.get_modules()[0].infer(zd);      /* lives until the generator's next pass */
					losses.push_back(gan.get_modules()[1].train_batch(fake, zerod, bce, CATTLE_HIP_OPT_ADAM, adam, 0, 2 * t));
					losses.push_back(gan.get_modules()[1].train_batch(reald, oned, bce, CATTLE_HIP_OPT_ADAM, adam, 0, 2 * t + 1));
					gan.get_modules()[1].set_frozen(true);
					losses.push_back(gan.train_batch(zd, oned, bce, CATTLE_HIP_OPT_ADAM, adam, 0, t));
					gan.get_modules()[1].set_frozen(false);
				}
				record_final<Scalar>(tag + ".gan1.g", gan.get_modules()[0]);
				record_final<Scalar>(tag + ".gan1.d", gan.get_modules()[1]);
			} else {
				DeviceFeedforwardNetwork<Scalar>& gen = nets[0];
				DeviceFeedforwardNetwork<Scalar>& disc = nets[1];
				for (std::size_t t = 0; t < 2; ++t) {
					const DT& fake = gen.propagate(zd, false);
					losses.push_back(disc.train_batch(fake, zerod, bce, CATTLE_HIP_OPT_ADAM, adam, 0, 2 * t));
					losses.push_back(disc.train_batch(reald, oned, bce, CATTLE_HIP_OPT_ADAM, adam, 0, 2 * t + 1));
					const DT& out = disc.propagate(gen.propagate(zd, true), true);
					Scalar total = 0;
					const std::vector<Scalar> per_sample = bce.function(out, oned);
					for (std::size_t i = 0; i < per_sample.size(); ++i)
						total += per_sample[i];
					losses.push_back(total);
					gen.backpropagate(disc.backpropagate(bce.d_function(out, oned, (Scalar) 1 / (Scalar) batch)));
					gen.optimizer_step(CATTLE_HIP_OPT_ADAM, adam, 0, t);
					disc.reset_grads();
				}
				record_final<Scalar>(tag + ".gan0.g", gen);
				record_final<Scalar>(tag + ".gan0.d", disc);
			}
			record(tag + ".gan" + std::to_string(stacked) + ".losses", sizeof(Scalar), { losses.size() }, losses.data());
		}
	}
	{
		/* NeuralNetwork::init with He initialization (as examples/cifar_convnet.cpp:21 sets it up): the weights must be
		 * what the reference's GaussianParameterInitialization::apply produces with the same standard library - a
		 * default-seeded engine per matrix, filled column by column - and the biases zero */
		std::vector<DL> layers;
		layers.push_back(DL::conv(Dims{ { 6, 6, 3 } }, 4));
		layers.push_back(DL::batch_norm(layers.back().get_output_dims()));
		layers.push_back(DL::trans_conv(layers.back().get_output_dims(), 2, 4, 4, 1, 1, 2, 2));
		layers.push_back(DL::dense(layers.back().get_output_dims(), 5));
		DeviceFeedforwardNetwork<Scalar> net(std::move(layers));
		net.init(HeParameterInitialization<Scalar>((Scalar) 1e-1));
		std::vector<Scalar> ok;
		for (std::size_t l = 0; l < net.get_layers().size(); ++l) {
			DL& layer = net.get_layers()[l];
			if (!layer.is_kernel_layer())
				continue;
			std::size_t rows, cols;
			bool optimizable;
			layer.param_shape(0, rows, cols, optimizable);
			std::default_random_engine gen;
			std::normal_distribution<Scalar> dist(0, (Scalar) 1e-1 * std::sqrt(2 / (Scalar) rows));
			std::vector<Scalar> want(rows * cols);
			for (std::size_t i = 0; i < cols; ++i)
				for (std::size_t j = 0; j < rows; ++j)
					want[j + rows * i] = dist(gen);
			ok.push_back(layer.get_param_values(0) == want ? (Scalar) 1 : (Scalar) 0);
			const std::vector<Scalar> bias = layer.get_param_values(1);
			Scalar nonzero = 0;
			for (std::size_t i = 0; i < bias.size(); ++i)
				nonzero += bias[i] != 0;
			ok.push_back(nonzero == 0 ? (Scalar) 1 : (Scalar) 0);
			record(tag + ".init_he.w" + std::to_string(l), sizeof(Scalar), { rows, cols }, want.data());
		}
		/* batch norm is no kernel layer: its first optimizable parameter, gamma, keeps its ones */
		Scalar gamma_ok = 0;
		for (std::size_t i = 0; i < net.get_layers()[1].num_params(); ++i) {
			std::size_t rows, cols;
			bool optimizable;
			net.get_layers()[1].param_shape(i, rows, cols, optimizable);
			if (optimizable) {
				const std::vector<Scalar> gamma = net.get_layers()[1].get_param_values(i);
				gamma_ok = gamma[0] == 1 && gamma[gamma.size() - 1] == 1 ? (Scalar) 1 : (Scalar) 0;
				break;
			}
		}
		ok.push_back(gamma_ok);
		record(tag + ".init_he.ok", sizeof(Scalar), { ok.size() }, ok.data());
		const Dims out_dims = net.get_layers()[2].get_output_dims();
		const std::vector<Scalar> dims = { (Scalar) out_dims[0], (Scalar) out_dims[1], (Scalar) out_dims[2] };
		record(tag + ".init_he.transconv_dims", sizeof(Scalar), { 3 }, dims.data());
	}
	{
		/* another loss of the loss/ directory, wrapped as NegatedLoss wraps it */
		Lcg g(13);
		const std::size_t batch = 9, classes = 7;
		std::vector<Scalar> o = random_values<Scalar>(batch * classes, g, 1.0), y = one_hot<Scalar>(batch, classes, g);
		DT od(typename DT::Dims{ { batch, classes, 1, 1 } }, o.data()), yd(typename DT::Dims{ { batch, classes, 1, 1 } }, y.data());
		DeviceLoss<Scalar> negated_hinge(CATTLE_HIP_LOSS_SQUARED_HINGE, (Scalar) 1e-5, true);
		record(tag + ".loss.out", sizeof(Scalar), { batch, classes }, o.data());
		record(tag + ".loss.obj", sizeof(Scalar), { batch, classes }, y.data());
		record(tag + ".loss.values", sizeof(Scalar), { batch }, negated_hinge.function(od, yd).data());
		record(tag + ".loss.grad", sizeof(Scalar), { batch, classes }, negated_hinge.d_function(od, yd, (Scalar) 0.5).to_host().data());
	}
	for (int fused = 0; fused < 2; ++fused) {
		const std::string convnet = tag + (fused ? ".convnetf" : ".convnet");
		Lcg g(12);
		const std::size_t batch = 16;
		std::vector<DL> layers;
		layers.push_back(DL::conv(Dims{ { 8, 8, 3 } }, 8));
		layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, layers.back().get_output_dims()));
		layers.push_back(DL::pool(CATTLE_HIP_POOL_MAX, layers.back().get_output_dims()));
		layers.push_back(DL::batch_norm(layers.back().get_output_dims()));
		layers.push_back(DL::dense(layers.back().get_output_dims(), 5));
		DeviceFeedforwardNetwork<Scalar> net(std::move(layers));
		if (fused) {
			const Scalar groups = (Scalar) net.fuse();
			record(convnet + ".groups", sizeof(Scalar), { 1 }, &groups);
		}
		init_and_record<Scalar>(convnet, net, g);
		std::vector<Scalar> x = random_values<Scalar>(batch * 8 * 8 * 3, g, 1.0), y = one_hot<Scalar>(batch, 5, g);
		record(convnet + ".x", sizeof(Scalar), { batch, 8, 8, 3 }, x.data());
		record(convnet + ".y", sizeof(Scalar), { batch, 5 }, y.data());
		DT xd(typename DT::Dims{ { batch, 8, 8, 3 } }, x.data()), yd(typename DT::Dims{ { batch, 5, 1, 1 } }, y.data());
		std::vector<Scalar> totals;
		for (std::size_t t = 0; t < steps; ++t)
			totals.push_back(net.train_batch_adam(xd, yd, loss, t, (Scalar) 0.01));
		record(convnet + ".losses", sizeof(Scalar), { steps }, totals.data());
		record_final<Scalar>(convnet, net);
		/* inference after training uses the running statistics */
		const DT& out = net.propagate(xd, false);
		record(convnet + ".infer", sizeof(Scalar), { batch, 5 }, out.to_host().data());
		/* the reference's parameter files: written, then read back by a fresh network, which must infer alike */
		net.save_all_unique_params_values(g_dir, tag + (fused ? "_fparams_" : "_params_"));
		std::vector<DL> twin_layers;
		twin_layers.push_back(DL::conv(Dims{ { 8, 8, 3 } }, 8));
		twin_layers.push_back(DL::activation(CATTLE_HIP_ACT_RELU, twin_layers.back().get_output_dims()));
		twin_layers.push_back(DL::pool(CATTLE_HIP_POOL_MAX, twin_layers.back().get_output_dims()));
		twin_layers.push_back(DL::batch_norm(twin_layers.back().get_output_dims()));
		twin_layers.push_back(DL::dense(twin_layers.back().get_output_dims(), 5));
		DeviceFeedforwardNetwork<Scalar> twin(std::move(twin_layers));
		twin.load_all_unique_params_values(g_dir, tag + (fused ? "_fparams_" : "_params_"));
		const DT& out2 = twin.propagate(xd, false);
		record(convnet + ".reloaded_infer", sizeof(Scalar), { batch, 5 }, out2.to_host().data());
	}
}

static std::pair<std::size_t,std::size_t> last_two_steps(std::size_t input_seq_length) {
	return std::make_pair((std::size_t) 2, input_seq_length - 2);
}

/* ConvLSTM: 4 steps of 5x4x3 input, 6 hidden channels, output = the last two hidden states, one SGD update. */
template<typename Scalar>
static void run_lstm(const std::string& tag) {
	typedef DeviceConvLSTM<Scalar> Net;
	Lcg g(13);
	const std::size_t batch = 8, T = 4, H = 5, W = 4, C = 3, hid = 6;
	Net net(typename Net::Dims{ { H, W, C } }, hid, &last_two_steps, false);
	for (int k = 0; k < 8; ++k) {
		const typename Net::Kernel kernel = (typename Net::Kernel) k;
		const std::size_t rows = net.kernel_size(kernel, false) / hid;
		std::vector<Scalar> w = random_values<Scalar>(rows * hid, g, std::sqrt(3.0 / (double) rows));
		std::vector<Scalar> b = random_values<Scalar>(hid, g, 0.1);
		net.set_kernel_values(kernel, false, w.data());
		net.set_kernel_values(kernel, true, b.data());
		record(tag + ".lstm.w" + std::to_string(k), sizeof(Scalar), { rows, hid }, w.data());
		record(tag + ".lstm.b" + std::to_string(k), sizeof(Scalar), { 1, hid }, b.data());
	}
	std::vector<Scalar> x = random_values<Scalar>(batch * T * H * W * C, g, 1.0);
	std::vector<Scalar> go = random_values<Scalar>(batch * 2 * H * W * hid, g, 1.0);
	record(tag + ".lstm.x", sizeof(Scalar), { batch, T, H, W, C }, x.data());
	record(tag + ".lstm.go", sizeof(Scalar), { batch, 2, H, W, hid }, go.data());
	typename Net::Sequence in, og;
	in.dims = { { batch, T, H, W, C } };
	in.data = DeviceTensor<Scalar>(typename DeviceTensor<Scalar>::Dims{ { batch * T, H, W, C } }, x.data());
	og.dims = { { batch, 2, H, W, hid } };
	og.data = DeviceTensor<Scalar>(typename DeviceTensor<Scalar>::Dims{ { batch * 2, H, W, hid } }, go.data());
	typename Net::Sequence out = net.propagate(in, true);
	record(tag + ".lstm.out", sizeof(Scalar), { batch, 2, H, W, hid }, out.data.to_host().data());
	typename Net::Sequence dx = net.backpropagate(og);
	record(tag + ".lstm.dx", sizeof(Scalar), { batch, T, H, W, C }, dx.data.to_host().data());
	for (int k = 0; k < 8; ++k) {
		const typename Net::Kernel kernel = (typename Net::Kernel) k;
		const std::size_t rows = net.kernel_size(kernel, false) / hid;
		record(tag + ".lstm.dw" + std::to_string(k), sizeof(Scalar), { rows, hid }, net.get_kernel_grad(kernel, false).data());
		record(tag + ".lstm.db" + std::to_string(k), sizeof(Scalar), { 1, hid }, net.get_kernel_grad(kernel, true).data());
	}
	/* the parameter files of the network as it stands, loaded by a fresh one, give the same output */
	net.save_all_unique_params_values(g_dir, tag + "_lstm_params_");
	{
		Net fresh(typename Net::Dims{ { H, W, C } }, hid, &last_two_steps, false);
		fresh.load_all_unique_params_values(g_dir, tag + "_lstm_params_");
		typename Net::Sequence again = fresh.propagate(in, true);
		record(tag + ".lstm.out_reloaded", sizeof(Scalar), { batch, 2, H, W, hid }, again.data.to_host().data());
	}
	net.sgd_update((Scalar) 0.05);
	net.reset_grads();
	record(tag + ".lstm.w3_updated", sizeof(Scalar), { net.kernel_size(Net::OUTPUT_WRITE, false) / hid, hid },
			net.get_kernel_values(Net::OUTPUT_WRITE, false).data());
}

int main(int argc, char** argv) {
	if (argc != 3) {
		std::fprintf(stderr, "usage: %s <records file> <scratch directory>\n", argv[0]);
		return 2;
	}
	g_dir = argv[2];
	try {
		check(cattle_hip_init(0));
		g_out = std::fopen(argv[1], "wb");
		if (!g_out)
			throw std::runtime_error("cannot open the records file");
		run<float>("f32");
		run<double>("f64");
		run_lstm<float>("f32");
		run_lstm<double>("f64");
		std::fclose(g_out);
	} catch (const std::exception& e) {
		std::fprintf(stderr, "device_net_test: %s\n", e.what());
		return 1;
	}
	return 0;
}
