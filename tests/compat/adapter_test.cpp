/*
 * adapter_test.cpp — drives the header-only HIP layers (HIPLayers.hpp) through the cattle::Layer
 * interface exactly as a NeuralNetwork would (pass_forward / pass_back on host tensors, parameters
 * through Parameters::get_values / set_values / get_grad), and records every tensor to a file that
 * tests/test_gpu_adapters.py checks against the CPU oracle.
 *
 * Compiled against tests/compat/cattle_interface_double.hpp because C-ATTL3 itself cannot be built
 * here (its Eigen submodule is absent); with the real library on the include path the same source
 * compiles unchanged after dropping the CATTLE_HIP_CATTLE_HEADER definition.
 */
#define CATTLE_HIP_CATTLE_HEADER "cattle_interface_double.hpp"
#include "cattle_hip/HIPLayers.hpp"

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>

using namespace cattle;

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

template<typename Scalar, std::size_t R>
static void record(const std::string& name, const Tensor<Scalar,R>& t) {
	std::vector<std::size_t> dims(t.dimensions().begin(), t.dimensions().end());
	record(name, sizeof(Scalar), dims, t.data());
}

template<typename Scalar>
static void record(const std::string& name, const Matrix<Scalar>& m) {
	record(name, sizeof(Scalar), { m.rows(), m.cols() }, m.data());
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

template<typename Scalar, std::size_t R>
static Tensor<Scalar,R> random_tensor(const std::array<std::size_t,R>& dims, Lcg& g, double scale = 1.0) {
	Tensor<Scalar,R> t(dims);
	for (std::size_t i = 0; i < t.size(); ++i)
		t.data()[i] = (Scalar) (g.next() * scale);
	return t;
}

template<typename Scalar>
static void randomize(Parameters<Scalar>& p, Lcg& g, double scale, double offset = 0.0) {
	Matrix<Scalar> m(p.get_rows(), p.get_cols());
	for (std::size_t i = 0; i < m.size(); ++i)
		m.data()[i] = (Scalar) (g.next() * scale + offset);
	p.set_values(m);
}

template<typename Scalar, std::size_t Rank>
static void init_params(Layer<Scalar,Rank>& layer) {
	for (Parameters<Scalar>* p : layer.get_params())
		p->init();                          /* what NeuralNetwork::init() does (core/NeuralNetwork.hpp:173-176) */
}

template<typename Scalar>
static void run(const std::string& tag) {
	typedef std::unique_ptr<Layer<Scalar,3>> LayerPtr3;
	Lcg g(sizeof(Scalar) == 4 ? 41 : 42);
	const std::size_t N = 6;

	/* 1. convolution: 3x2 receptor, padding (1,2), stride (1,2), dilation (1,0) as in test/gradient_test.cpp:175 */
	{
		hip::ConvKernelHIPLayer<Scalar,3> conv({ 8u, 8u, 2u }, 5, nullptr, 3, 2, 1, 2, 1, 2, 1, 0);
		init_params(conv);
		randomize(*conv.get_params()[0], g, 0.5);
		randomize(*conv.get_params()[1], g, 0.5);
		auto x = random_tensor<Scalar,4>({ { N, 8, 8, 2 } }, g);
		record(tag + "conv.x", x);
		record(tag + "conv.w", conv.get_params()[0]->get_values());
		record(tag + "conv.b", conv.get_params()[1]->get_values());
		auto out = conv.pass_forward(x, true);
		record(tag + "conv.out", out);
		auto go = random_tensor<Scalar,4>(out.dimensions(), g);
		record(tag + "conv.go", go);
		auto dx = conv.pass_back(go);
		record(tag + "conv.dx", dx);
		record(tag + "conv.dw", conv.get_params()[0]->get_grad());
		record(tag + "conv.db", conv.get_params()[1]->get_grad());
		/* a second pass_back accumulates into the same Parameters; a shared-parameter clone does too */
		conv.pass_back(go);
		std::unique_ptr<Layer<Scalar,3>> twin(conv.clone_with_shared_params());
		if (!twin->is_shared_params_clone() || twin->get_params()[0] != conv.get_params()[0])
			throw std::runtime_error("clone_with_shared_params does not share the parameters");
		twin->set_input_layer(true);
		twin->pass_forward(x, true);
		auto none = twin->pass_back(go);
		if (none.size() != 0)
			throw std::runtime_error("an input layer must return a null tensor from pass_back");
		record(tag + "conv.dw3", conv.get_params()[0]->get_grad());
		std::unique_ptr<Layer<Scalar,3>> deep(conv.clone());
		if (deep->is_shared_params_clone() || deep->get_params()[0] == conv.get_params()[0])
			throw std::runtime_error("clone must copy the parameters");
	}
	/* 1b. transposed convolution, the rank-3 geometry of test/gradient_test.cpp:201, and its rank-1 form (:194) */
	{
		hip::TransConvKernelHIPLayer<Scalar,3> trans({ 2u, 3u, 2u }, 5, nullptr, 5, 3, 1, 0, 1, 2, 0, 1);
		init_params(trans);
		randomize(*trans.get_params()[0], g, 0.5);
		randomize(*trans.get_params()[1], g, 0.5);
		if (trans.get_output_dims()(0) != 4 || trans.get_output_dims()(1) != 9 || trans.get_output_dims()(2) != 5)
			throw std::runtime_error("transposed convolution output dims");
		auto x = random_tensor<Scalar,4>({ { N, 2, 3, 2 } }, g);
		record(tag + "trans.x", x);
		record(tag + "trans.w", trans.get_params()[0]->get_values());
		record(tag + "trans.b", trans.get_params()[1]->get_values());
		auto out = trans.pass_forward(x, true);
		record(tag + "trans.out", out);
		auto go = random_tensor<Scalar,4>(out.dimensions(), g);
		record(tag + "trans.go", go);
		record(tag + "trans.dx", trans.pass_back(go));
		record(tag + "trans.dw", trans.get_params()[0]->get_grad());
		record(tag + "trans.db", trans.get_params()[1]->get_grad());
		hip::TransConvKernelHIPLayer<Scalar,1> trans1({ 16u }, 5, nullptr, 4, 1, 1, 1);
		init_params(trans1);
		randomize(*trans1.get_params()[0], g, 0.5);
		if (trans1.get_output_dims()(0) != 100)
			throw std::runtime_error("rank-1 transposed convolution output dims");
		auto x1 = random_tensor<Scalar,2>({ { N, 16 } }, g);
		record(tag + "trans1.x", x1);
		record(tag + "trans1.w", trans1.get_params()[0]->get_values());
		record(tag + "trans1.out", trans1.pass_forward(x1, true));
	}
	/* 2. dense on rank-3 data */
	{
		hip::DenseKernelHIPLayer<Scalar,3> dense({ 4u, 4u, 2u }, 16, nullptr);
		init_params(dense);
		randomize(*dense.get_params()[0], g, 0.3);
		randomize(*dense.get_params()[1], g, 0.3);
		auto x = random_tensor<Scalar,4>({ { N, 4, 4, 2 } }, g);
		record(tag + "dense.x", x);
		record(tag + "dense.w", dense.get_params()[0]->get_values());
		record(tag + "dense.b", dense.get_params()[1]->get_values());
		auto out = dense.pass_forward(x, true);
		record(tag + "dense.out", out);
		auto go = random_tensor<Scalar,4>(out.dimensions(), g);
		record(tag + "dense.go", go);
		record(tag + "dense.dx", dense.pass_back(go));
		record(tag + "dense.dw", dense.get_params()[0]->get_grad());
		record(tag + "dense.db", dense.get_params()[1]->get_grad());
		/* the layer uploads a parameter only when its host values changed: unchanged values give the same output again,
		 * values set through the Parameters object (what an optimizer does) show in the next pass */
		auto again = dense.pass_forward(x, false);
		for (std::size_t i = 0; i < out.size(); ++i)
			if (again.data()[i] != out.data()[i])
				throw std::runtime_error("a second pass with unchanged parameters differs");
		randomize(*dense.get_params()[0], g, 0.3);
		randomize(*dense.get_params()[1], g, 0.3);
		record(tag + "dense.w2", dense.get_params()[0]->get_values());
		record(tag + "dense.b2", dense.get_params()[1]->get_values());
		record(tag + "dense.out2", dense.pass_forward(x, false));
	}
	/* 3. batch norm per channel: two training passes, then inference */
	{
		hip::BatchNormHIPLayer<Scalar,3> bn({ 5u, 4u, 3u }, (Scalar) 0.2);
		init_params(bn);
		auto params = bn.get_params();
		if (params.size() != 12 || params[0]->are_optimizable() || !params[2]->are_optimizable() ||
				params[2]->get_values()(0, 0) != 1 || params[3]->get_values()(0, 0) != 0)
			throw std::runtime_error("batch norm parameters are not laid out like the reference's");
		Matrix<Scalar> gamma(1, 3), beta(1, 3);
		for (std::size_t c = 0; c < 3; ++c) {
			randomize(*params[4 * c + 2], g, 0.3, 1.0);
			randomize(*params[4 * c + 3], g, 0.3);
			gamma(0, c) = params[4 * c + 2]->get_values()(0, 0);
			beta(0, c) = params[4 * c + 3]->get_values()(0, 0);
		}
		record(tag + "bn.gamma", gamma);
		record(tag + "bn.beta", beta);
		auto x1 = random_tensor<Scalar,4>({ { N, 5, 4, 3 } }, g, 2.0);
		auto x2 = random_tensor<Scalar,4>({ { N, 5, 4, 3 } }, g, 0.5);
		record(tag + "bn.x1", x1);
		record(tag + "bn.x2", x2);
		record(tag + "bn.y1", bn.pass_forward(x1, true));
		auto go = random_tensor<Scalar,4>(x1.dimensions(), g);
		record(tag + "bn.go", go);
		record(tag + "bn.dx1", bn.pass_back(go));
		Matrix<Scalar> dgamma(1, 3), dbeta(1, 3), mean(1, 3), inv_sd(1, 3);
		for (std::size_t c = 0; c < 3; ++c) {
			dgamma(0, c) = params[4 * c + 2]->get_grad()(0, 0);
			dbeta(0, c) = params[4 * c + 3]->get_grad()(0, 0);
		}
		record(tag + "bn.dgamma", dgamma);
		record(tag + "bn.dbeta", dbeta);
		bn.pass_forward(x2, true);
		for (std::size_t c = 0; c < 3; ++c) {
			mean(0, c) = params[4 * c]->get_values()(0, 0);
			inv_sd(0, c) = params[4 * c + 1]->get_values()(0, 0);
		}
		record(tag + "bn.avg_mean", mean);
		record(tag + "bn.avg_inv_sd", inv_sd);
		record(tag + "bn.y_infer", bn.pass_forward(x1, false));
	}
	/* 4. activations */
	{
		auto x = random_tensor<Scalar,4>({ { N, 3, 5, 2 } }, g, 2.0);
		auto go = random_tensor<Scalar,4>(x.dimensions(), g);
		record(tag + "act.x", x);
		record(tag + "act.go", go);
		typename Layer<Scalar,3>::PublicDims dims({ 3u, 5u, 2u });
		std::vector<std::pair<std::string,LayerPtr3>> acts;
		acts.emplace_back("relu", LayerPtr3(new hip::ReLUActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("sigmoid", LayerPtr3(new hip::SigmoidActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("tanh", LayerPtr3(new hip::TanhActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("leaky_relu", LayerPtr3(new hip::LeakyReLUActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("elu", LayerPtr3(new hip::ELUActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("swish", LayerPtr3(new hip::SwishActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("softplus", LayerPtr3(new hip::SoftplusActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("softsign", LayerPtr3(new hip::SoftsignActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("identity", LayerPtr3(new hip::IdentityActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("scaled", LayerPtr3(new hip::ScaledActivationHIPLayer<Scalar,3>(dims, (Scalar) 1.5)));
		acts.emplace_back("binary_step", LayerPtr3(new hip::BinaryStepActivationHIPLayer<Scalar,3>(dims)));
		acts.emplace_back("softmax", LayerPtr3(new hip::SoftmaxActivationHIPLayer<Scalar,3>(dims)));
		for (auto& a : acts) {
			record(tag + "act." + a.first + ".y", a.second->pass_forward(x, true));
			record(tag + "act." + a.first + ".dx", a.second->pass_back(go));
			std::unique_ptr<Layer<Scalar,3>> c(a.second->clone());
			record(tag + "act." + a.first + ".y_clone", c->pass_forward(x, true));
		}
		hip::PReLUActivationHIPLayer<Scalar,3> prelu(dims);
		init_params(prelu);
		if (prelu.get_params()[0]->get_values()(0, 7) != (Scalar) 1e-1)
			throw std::runtime_error("PReLU alpha is not initialised to init_alpha");
		randomize(*prelu.get_params()[0], g, 0.4, 0.6);
		record(tag + "act.prelu.alpha", prelu.get_params()[0]->get_values());
		record(tag + "act.prelu.y", prelu.pass_forward(x, true));
		record(tag + "act.prelu.dx", prelu.pass_back(go));
		record(tag + "act.prelu.dalpha", prelu.get_params()[0]->get_grad());
	}
	/* 5. pooling, rank 3 and rank 1 */
	{
		auto x = random_tensor<Scalar,4>({ { N, 16, 16, 2 } }, g);
		record(tag + "pool.x", x);
		hip::MaxPoolHIPLayer<Scalar,3> mx({ 16u, 16u, 2u }, 3, 2, 1, 2);         /* test/gradient_test.cpp:313 */
		auto out = mx.pass_forward(x, true);
		record(tag + "pool.max.out", out);
		std::vector<unsigned> inds = mx.get_max_indices();
		record(tag + "pool.max.inds", 4, { inds.size() }, inds.data());
		auto go = random_tensor<Scalar,4>(out.dimensions(), g);
		record(tag + "pool.go", go);
		record(tag + "pool.max.dx", mx.pass_back(go));
		hip::MeanPoolHIPLayer<Scalar,3> mn({ 16u, 16u, 2u }, 3, 2, 1, 2);
		record(tag + "pool.mean.out", mn.pass_forward(x, true));
		record(tag + "pool.mean.dx", mn.pass_back(go));
		hip::MaxPoolHIPLayer<Scalar,1> m1({ 32u }, 3, 1);                        /* test/gradient_test.cpp:299 */
		auto x1 = random_tensor<Scalar,2>({ { N, 32 } }, g);
		record(tag + "pool1.x", x1);
		record(tag + "pool1.out", m1.pass_forward(x1, true));
	}
	/* 6. a small feed-forward stack driven the way FeedforwardNeuralNetwork does it
	 * (neural_network/FeedforwardNeuralNetwork.hpp:38-53, :112-127): layer 0 is the input layer */
	{
		std::vector<LayerPtr3> net;
		net.emplace_back(new hip::ConvKernelHIPLayer<Scalar,3>({ 8u, 8u, 3u }, 4, nullptr));
		net.emplace_back(new hip::ReLUActivationHIPLayer<Scalar,3>(net.back()->get_output_dims()));
		net.emplace_back(new hip::MaxPoolHIPLayer<Scalar,3>(net.back()->get_output_dims()));
		net.emplace_back(new hip::ConvKernelHIPLayer<Scalar,3>(net.back()->get_output_dims(), 6, nullptr));
		net.emplace_back(new hip::BatchNormHIPLayer<Scalar,3>(net.back()->get_output_dims()));
		net.emplace_back(new hip::ReLUActivationHIPLayer<Scalar,3>(net.back()->get_output_dims()));
		net.emplace_back(new hip::MaxPoolHIPLayer<Scalar,3>(net.back()->get_output_dims()));
		net.emplace_back(new hip::DenseKernelHIPLayer<Scalar,3>(net.back()->get_output_dims(), 10, nullptr));
		net[0]->set_input_layer(true);
		for (auto& l : net)
			init_params(*l);
		randomize(*net[0]->get_params()[0], g, 0.3);
		randomize(*net[3]->get_params()[0], g, 0.2);
		randomize(*net[7]->get_params()[0], g, 0.2);
		record(tag + "net.w0", net[0]->get_params()[0]->get_values());
		record(tag + "net.w3", net[3]->get_params()[0]->get_values());
		record(tag + "net.w7", net[7]->get_params()[0]->get_values());
		auto x = random_tensor<Scalar,4>({ { N, 8, 8, 3 } }, g);
		record(tag + "net.x", x);
		auto h = x;
		for (auto& l : net)
			h = l->pass_forward(std::move(h), true);
		record(tag + "net.out", h);
		auto grad = random_tensor<Scalar,4>(h.dimensions(), g);
		record(tag + "net.go", grad);
		for (std::size_t i = net.size(); i-- > 0;)
			grad = net[i]->pass_back(std::move(grad));
		if (grad.size() != 0)
			throw std::runtime_error("the input layer must not produce an input gradient");
		record(tag + "net.dw0", net[0]->get_params()[0]->get_grad());
		record(tag + "net.db0", net[0]->get_params()[1]->get_grad());
		record(tag + "net.dw3", net[3]->get_params()[0]->get_grad());
		record(tag + "net.dw7", net[7]->get_params()[0]->get_grad());
	}
}

int main(int argc, char** argv) {
	if (argc < 2) {
		std::fprintf(stderr, "usage: %s <output file>\n", argv[0]);
		return 2;
	}
	g_out = std::fopen(argv[1], "wb");
	if (!g_out)
		return 2;
	try {
		run<float>("f32.");
		run<double>("f64.");
	} catch (const std::exception& e) {
		std::fprintf(stderr, "adapter_test failed: %s\n", e.what());
		std::fclose(g_out);
		return 1;
	}
	std::fclose(g_out);
	std::printf("adapter_test: ok\n");
	return 0;
}
