/*
 * DeviceNet.hpp — header-only C++11 view of libcattle_hip for callers that keep a whole training
 * step on the MI355X: device tensors chained from layer to layer, parameters that never leave the
 * device, loss and optimizer update as kernels.
 *
 * It plays the part that core/gpu/GPULayer.hpp:31-58, core/gpu/GPUNeuralNetwork.hpp:27-48 and
 * parameters/gpu/StandardGPUParameters.hpp:50-120 sketch in the reference's unfinished CUDA tree
 * (device-tensor overloads of pass_forward / pass_back / propagate / backpropagate, device-side
 * values and gradients), and the training loop is SGDOptimizer::_train's batch body
 * (optimizer/SGDOptimizer.hpp:44-70). It needs no C-ATTL3 header: only the C ABI.
 *
 * Tensors are the reference's column-major buffers with the sample index fastest; dims are
 * (batch, height, width, channels) the way Dimensions::extend pads lower ranks with ones.
 */
#ifndef CATTLE_HIP_DEVICENET_HPP_
#define CATTLE_HIP_DEVICENET_HPP_

#include <array>
#include <cassert>
#include <cstddef>
#include <fstream>
#include <cmath>
#include <memory>
#include <random>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "cattle_hip.h"

namespace cattle {
namespace hip {
namespace device {

inline void check(int status) {
	if (status != CATTLE_HIP_OK)
		throw std::runtime_error(std::string("cattle_hip: ") + cattle_hip_last_error());
}

template<typename Scalar> struct Code;
template<> struct Code<float> { static constexpr cattle_hip_dtype value = CATTLE_HIP_F32; };
template<> struct Code<double> { static constexpr cattle_hip_dtype value = CATTLE_HIP_F64; };

/**
 * The parameter initializations of the parameter_initialization/ headers on a column-major host matrix (the values are
 * uploaded by DeviceLayer::init_params). They use the standard library exactly as the reference does - a default-seeded
 * std::default_random_engine per matrix and std::normal_distribution, filled column by column
 * (GaussianParameterInitialization.hpp:34-44) - so a build against the same standard library starts from the reference's
 * initial values.
 */
template<typename Scalar>
class ParameterInitialization {
public:
	virtual ~ParameterInitialization() { }
	virtual void apply(std::vector<Scalar>& values, std::size_t rows, std::size_t cols) const = 0;
};

/** parameter_initialization/GaussianParameterInitialization.hpp:28-52 */
template<typename Scalar>
class GaussianParameterInitialization : public ParameterInitialization<Scalar> {
public:
	inline GaussianParameterInitialization(Scalar mean = 0, Scalar sd_scaling_factor = 1) : mean(mean),
			sd_scaling_factor(sd_scaling_factor) {
		assert(sd_scaling_factor > 0);
	}
	inline void apply(std::vector<Scalar>& values, std::size_t rows, std::size_t cols) const {
		std::default_random_engine gen;
		std::normal_distribution<Scalar> dist(mean, sd_scaling_factor * _sd((unsigned) rows, (unsigned) cols));
		values.resize(rows * cols);
		for (std::size_t i = 0; i < cols; ++i)
			for (std::size_t j = 0; j < rows; ++j)
				values[j + rows * i] = dist(gen);
	}
protected:
	inline virtual Scalar _sd(unsigned fan_ins, unsigned fan_outs) const {
		return 1;
	}
private:
	const Scalar mean, sd_scaling_factor;
};

/** parameter_initialization/HeParameterInitialization.hpp:27-36 */
template<typename Scalar>
class HeParameterInitialization : public GaussianParameterInitialization<Scalar> {
public:
	inline HeParameterInitialization(Scalar sd_scaling_factor = 1) : GaussianParameterInitialization<Scalar>(0, sd_scaling_factor) { }
protected:
	inline Scalar _sd(unsigned fan_ins, unsigned fan_outs) const {
		return std::sqrt(2 / (Scalar) fan_ins);
	}
};

/** parameter_initialization/GlorotParameterInitialization.hpp:27-36 */
template<typename Scalar>
class GlorotParameterInitialization : public GaussianParameterInitialization<Scalar> {
public:
	inline GlorotParameterInitialization(Scalar sd_scaling_factor = 1) : GaussianParameterInitialization<Scalar>(0, sd_scaling_factor) { }
protected:
	inline Scalar _sd(unsigned fan_ins, unsigned fan_outs) const {
		return std::sqrt(2 / (Scalar) (fan_ins + fan_outs));
	}
};

/** parameter_initialization/LeCunParameterInitialization.hpp:27-36 */
template<typename Scalar>
class LeCunParameterInitialization : public GaussianParameterInitialization<Scalar> {
public:
	inline LeCunParameterInitialization(Scalar sd_scaling_factor = 1) : GaussianParameterInitialization<Scalar>(0, sd_scaling_factor) { }
protected:
	inline Scalar _sd(unsigned fan_ins, unsigned fan_outs) const {
		return std::sqrt(1 / (Scalar) fan_ins);
	}
};

/** parameter_initialization/ConstantParameterInitialization.hpp:24-33 (Zero and One are its 0 and 1) */
template<typename Scalar>
class ConstantParameterInitialization : public ParameterInitialization<Scalar> {
public:
	inline ConstantParameterInitialization(Scalar constant) : constant(constant) { }
	inline void apply(std::vector<Scalar>& values, std::size_t rows, std::size_t cols) const {
		values.assign(rows * cols, constant);
	}
private:
	const Scalar constant;
};

/** parameter_initialization/IncrementalParameterInitialization.hpp:24-42 */
template<typename Scalar>
class IncrementalParameterInitialization : public ParameterInitialization<Scalar> {
public:
	inline IncrementalParameterInitialization(Scalar start, Scalar inc) : start(start), inc(inc) { }
	inline void apply(std::vector<Scalar>& values, std::size_t rows, std::size_t cols) const {
		values.resize(rows * cols);
		Scalar val = start;
		for (std::size_t i = 0; i < cols; ++i)
			for (std::size_t j = 0; j < rows; ++j) {
				values[j + rows * i] = val;
				val += inc;
			}
	}
private:
	const Scalar start, inc;
};

/** A tensor in device memory; move-only owner of its buffer (the role of CuDNNTensor in the reference). */
template<typename Scalar>
class DeviceTensor {
public:
	typedef std::array<std::size_t,4> Dims;
	inline DeviceTensor() : dims{ { 0, 0, 0, 0 } }, ptr(nullptr) { }
	inline explicit DeviceTensor(const Dims& dims) : dims(dims), ptr(nullptr) {
		if (size() > 0)
			check(cattle_hip_alloc(&ptr, size() * sizeof(Scalar)));
	}
	/** Uploads a host buffer of the same layout (an Eigen tensor's data()). */
	inline DeviceTensor(const Dims& dims, const Scalar* host) : DeviceTensor(dims) {
		if (size() > 0)
			check(cattle_hip_upload(ptr, host, size() * sizeof(Scalar)));
	}
	inline DeviceTensor(DeviceTensor&& other) : dims(other.dims), ptr(other.ptr) {
		other.ptr = nullptr;
		other.dims = Dims{ { 0, 0, 0, 0 } };
	}
	inline DeviceTensor& operator=(DeviceTensor&& other) {
		if (this != &other) {
			release();
			dims = other.dims;
			ptr = other.ptr;
			other.ptr = nullptr;
			other.dims = Dims{ { 0, 0, 0, 0 } };
		}
		return *this;
	}
	DeviceTensor(const DeviceTensor&) = delete;
	DeviceTensor& operator=(const DeviceTensor&) = delete;
	inline ~DeviceTensor() {
		release();
	}
	inline std::size_t size() const {
		return dims[0] * dims[1] * dims[2] * dims[3];
	}
	inline std::size_t batch() const {
		return dims[0];
	}
	inline const Dims& dimensions() const {
		return dims;
	}
	/** A null tensor, as pass_back of an input layer returns (core/Layer.hpp:131-137). */
	inline bool is_null() const {
		return ptr == nullptr;
	}
	inline Scalar* data() {
		return static_cast<Scalar*>(ptr);
	}
	inline const Scalar* data() const {
		return static_cast<const Scalar*>(ptr);
	}
	inline void download(Scalar* host) const {
		if (size() > 0)
			check(cattle_hip_download(host, ptr, size() * sizeof(Scalar)));
	}
	inline std::vector<Scalar> to_host() const {
		std::vector<Scalar> out(size());
		download(out.data());
		return out;
	}
private:
	inline void release() {
		if (ptr)
			cattle_hip_free(ptr);
		ptr = nullptr;
	}
	Dims dims;
	void* ptr;
};

/** One layer on the device: owner of a cattle_hip_layer_t, with the Layer contract on DeviceTensors. */
template<typename Scalar>
class DeviceLayer {
public:
	typedef std::array<std::size_t,3> Dims;
	/* layer/kernel/ConvKernelLayer.hpp:282-296 */
	inline static DeviceLayer conv(const Dims& input_dims, std::size_t filters, std::size_t receptor_height = 3,
			std::size_t receptor_width = 3, std::size_t vertical_padding = 1, std::size_t horizontal_padding = 1,
			std::size_t vertical_stride = 1, std::size_t horizontal_stride = 1, std::size_t vertical_dilation = 0,
			std::size_t horizontal_dilation = 0) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_conv_create(Code<Scalar>::value, input_dims[0], input_dims[1], input_dims[2], filters,
				receptor_height, receptor_width, vertical_padding, horizontal_padding, vertical_stride, horizontal_stride,
				vertical_dilation, horizontal_dilation, &h));
		DeviceLayer layer(h);
		layer.kernel_layer = true;
		return layer;
	}
	/* layer/kernel/TransConvKernelLayer.hpp:290-304 */
	inline static DeviceLayer trans_conv(const Dims& input_dims, std::size_t filters, std::size_t receptor_height = 3,
			std::size_t receptor_width = 3, std::size_t vertical_padding = 1, std::size_t horizontal_padding = 1,
			std::size_t vertical_stride = 1, std::size_t horizontal_stride = 1, std::size_t vertical_dilation = 0,
			std::size_t horizontal_dilation = 0) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_transconv_create(Code<Scalar>::value, input_dims[0], input_dims[1], input_dims[2], filters,
				receptor_height, receptor_width, vertical_padding, horizontal_padding, vertical_stride, horizontal_stride,
				vertical_dilation, horizontal_dilation, &h));
		DeviceLayer layer(h);
		layer.kernel_layer = true;
		return layer;
	}
	/* layer/kernel/DenseKernelLayer.hpp:61-77 */
	inline static DeviceLayer dense(const Dims& input_dims, std::size_t output_size) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_dense_create(Code<Scalar>::value, input_dims[0] * input_dims[1] * input_dims[2], output_size, &h));
		DeviceLayer layer(h, input_dims);
		layer.kernel_layer = true;
		return layer;
	}
	/* layer/BatchNormLayer.hpp:66-101 (per channel) / :334-361 (per activation) */
	inline static DeviceLayer batch_norm(const Dims& dims, bool per_last_rank = true, Scalar norm_avg_decay = .1,
			Scalar epsilon = 1e-5) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_batchnorm_create(Code<Scalar>::value, dims[0], dims[1], dims[2], per_last_rank ? 1 : 0,
				(double) norm_avg_decay, (double) epsilon, &h));
		DeviceLayer layer(h);
		layer.params_per_column = per_last_rank;
		return layer;
	}
	/* layer/activation/<Name>ActivationLayer.hpp */
	inline static DeviceLayer activation(cattle_hip_activation kind, const Dims& dims, Scalar param = 0) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_activation_create(Code<Scalar>::value, kind, dims[0] * dims[1] * dims[2], (double) param, &h));
		return DeviceLayer(h, dims, dims);
	}
	/* layer/pool/MaxPoolLayer.hpp:105-108, layer/pool/MeanPoolLayer.hpp:62-65 */
	inline static DeviceLayer pool(cattle_hip_pool kind, const Dims& input_dims, std::size_t receptor_height = 2,
			std::size_t receptor_width = 2, std::size_t vertical_stride = 2, std::size_t horizontal_stride = 2) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_pool_create(Code<Scalar>::value, kind, input_dims[0], input_dims[1], input_dims[2], receptor_height,
				receptor_width, vertical_stride, horizontal_stride, &h));
		return DeviceLayer(h);
	}
	/* layer/DropoutLayer.hpp:33-42; `seed` keys the generator of the masks (give every dropout layer its own) */
	inline static DeviceLayer dropout(const Dims& dims, Scalar dropout_prob, unsigned long long seed = 0, Scalar epsilon = 1e-5) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_dropout_create(Code<Scalar>::value, dims[0] * dims[1] * dims[2], (double) dropout_prob, (double) epsilon,
				seed, &h));
		return DeviceLayer(h, dims, dims);
	}
	/* layer/ReshapeLayer.hpp:31-39 */
	inline static DeviceLayer reshape(const Dims& input_dims, const Dims& output_dims) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_reshape_create(Code<Scalar>::value, input_dims.data(), output_dims.data(), &h));
		return DeviceLayer(h);
	}
	/* layer/BroadcastLayer.hpp:31-40 */
	inline static DeviceLayer broadcast(const Dims& input_dims, const Dims& broadcast) {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_broadcast_create(Code<Scalar>::value, input_dims.data(), broadcast.data(), &h));
		return DeviceLayer(h);
	}
	/**
	 * A kernel layer and the batch norm / activation / pool layers a network calls right after it as one layer
	 * (cattle_hip_fused_create): `members` = { convolutional or dense layer [, batch norm] [, activation] [, pool] } in
	 * call order. The members are borrowed (their parameters, running statistics and caches stay theirs) and must
	 * outlive the result. Returns a layer without a handle (is_null()) if these layers cannot form a fused layer.
	 */
	inline static DeviceLayer fused(const DeviceLayer* const* members, std::size_t count) {
		cattle_hip_layer_t handles[4] = { nullptr, nullptr, nullptr, nullptr };
		cattle_hip_layer_t h = nullptr;
		if (count < 2 || count > 4)
			return DeviceLayer(nullptr, Dims(), Dims());
		for (std::size_t i = 0; i < count; ++i)
			handles[i] = members[i]->handle;
		if (cattle_hip_fused_create(handles, count, &h) != CATTLE_HIP_OK)
			return DeviceLayer(nullptr, Dims(), Dims());
		return DeviceLayer(h, members[0]->in_dims, members[count - 1]->out_dims);
	}
	inline bool is_null() const {
		return handle == nullptr;
	}
	inline DeviceLayer(DeviceLayer&& other) : handle(other.handle), in_dims(other.in_dims), out_dims(other.out_dims),
			cached_in(std::move(other.cached_in)), cached_out(std::move(other.cached_out)),
			params_per_column(other.params_per_column), kernel_layer(other.kernel_layer) {
		other.handle = nullptr;
	}
	DeviceLayer(const DeviceLayer&) = delete;
	DeviceLayer& operator=(const DeviceLayer&) = delete;
	inline ~DeviceLayer() {
		if (handle)
			cattle_hip_layer_destroy(handle);
	}
	/* Layer::clone (core/Layer.hpp:47) / clone_with_shared_params (:56) */
	inline DeviceLayer clone(bool share_params = false) const {
		cattle_hip_layer_t h = nullptr;
		check(cattle_hip_layer_clone(handle, share_params ? 1 : 0, &h));
		return DeviceLayer(h, in_dims, out_dims);
	}
	inline const Dims& get_input_dims() const {
		return in_dims;
	}
	inline const Dims& get_output_dims() const {
		return out_dims;
	}
	inline bool is_input_layer() const {
		int flag = 0;
		check(cattle_hip_layer_is_input_layer(handle, &flag));
		return flag != 0;
	}
	inline void set_input_layer(bool input_layer) {
		check(cattle_hip_layer_set_input_layer(handle, input_layer ? 1 : 0));
	}
	inline void empty_cache() {
		check(cattle_hip_layer_empty_cache(handle));
		cached_in = DeviceTensor<Scalar>();
		cached_out = DeviceTensor<Scalar>();
	}
	/**
	 * Layer::pass_forward on device tensors. The layer borrows its input (and, for layers whose backward
	 * pass reads the output, its output) until pass_back, so the input is taken by value and kept here, and
	 * the returned reference stays valid until the next pass_forward or empty_cache of this layer.
	 */
	inline const DeviceTensor<Scalar>& pass_forward(DeviceTensor<Scalar> in, bool training) {
		assert(in.dimensions()[1] * in.dimensions()[2] * in.dimensions()[3] == in_dims[0] * in_dims[1] * in_dims[2]);
		const std::size_t batch = in.batch();
		DeviceTensor<Scalar> out(typename DeviceTensor<Scalar>::Dims{ { batch, out_dims[0], out_dims[1], out_dims[2] } });
		check(cattle_hip_layer_forward(handle, in.data(), CATTLE_HIP_DEVICE, batch, training ? 1 : 0, out.data(),
				CATTLE_HIP_DEVICE));
		cached_in = std::move(in);
		cached_out = std::move(out);
		return cached_out;
	}
	/** Same, for an input the caller keeps alive and unmodified until pass_back (e.g. the training batch). */
	inline const DeviceTensor<Scalar>& pass_forward_borrowed(const DeviceTensor<Scalar>& in, bool training) {
		const std::size_t batch = in.batch();
		DeviceTensor<Scalar> out(typename DeviceTensor<Scalar>::Dims{ { batch, out_dims[0], out_dims[1], out_dims[2] } });
		check(cattle_hip_layer_forward(handle, in.data(), CATTLE_HIP_DEVICE, batch, training ? 1 : 0, out.data(),
				CATTLE_HIP_DEVICE));
		cached_in = DeviceTensor<Scalar>();
		cached_out = std::move(out);
		return cached_out;
	}
	/** Layer::pass_back: returns the input gradient, a null tensor for an input layer. */
	inline DeviceTensor<Scalar> pass_back(const DeviceTensor<Scalar>& out_grad, bool needs_input_grad = true) {
		const std::size_t batch = out_grad.batch();
		DeviceTensor<Scalar> prev;
		if (needs_input_grad)
			prev = DeviceTensor<Scalar>(typename DeviceTensor<Scalar>::Dims{ { batch, in_dims[0], in_dims[1], in_dims[2] } });
		check(cattle_hip_layer_backward(handle, out_grad.data(), CATTLE_HIP_DEVICE, batch,
				needs_input_grad ? prev.data() : nullptr, CATTLE_HIP_DEVICE));
		return prev;
	}
	/* ---- parameters (core/Parameters.hpp:15-95), resident on the device ---- */
	inline std::size_t num_params() const {
		std::size_t n = 0;
		check(cattle_hip_layer_num_params(handle, &n));
		return n;
	}
	inline void param_shape(std::size_t index, std::size_t& rows, std::size_t& cols, bool& optimizable) const {
		int opt = 0;
		check(cattle_hip_layer_param_shape(handle, index, &rows, &cols, &opt));
		optimizable = opt != 0;
	}
	inline void set_param_values(std::size_t index, const Scalar* host_values) {
		check(cattle_hip_layer_set_param_values(handle, index, host_values, CATTLE_HIP_HOST));
	}
	inline std::vector<Scalar> get_param_values(std::size_t index) const {
		return fetch(index, &cattle_hip_layer_get_param_values);
	}
	inline std::vector<Scalar> get_param_grad(std::size_t index) const {
		return fetch(index, &cattle_hip_layer_get_param_grad);
	}
	/** Whether the layer is a kernel layer: parameter 0 its weight matrix, parameter 1 its bias. */
	inline bool is_kernel_layer() const {
		return kernel_layer;
	}
	/**
	 * Parameters::init_values (parameters/StandardParameters.hpp:91-95) for parameter `index`: the initialization applied
	 * to a host matrix of the parameter's shape and uploaded.
	 */
	inline void init_params(std::size_t index, const ParameterInitialization<Scalar>& init) {
		std::size_t rows, cols;
		bool optimizable;
		param_shape(index, rows, cols, optimizable);
		std::vector<Scalar> values;
		init.apply(values, rows, cols);
		set_param_values(index, values.data());
	}
	/**
	 * The ParameterRegularization of parameter `index` (the weight_reg / bias_reg arguments of the reference's kernel
	 * layers): L1 = (lambda, 0), L2 = (0, lambda), elastic net = (l1, l2). optimizer_step regularizes before it updates.
	 */
	inline void set_regularization(std::size_t index, Scalar l1_lambda, Scalar l2_lambda) {
		check(cattle_hip_layer_param_set_regularization(handle, index, (double) l1_lambda, (double) l2_lambda));
	}
	/**
	 * The value and gradient constraints of parameter `index` (the weight_clip, weight_max_l1_norm, weight_max_l2_norm,
	 * weight_grad_clip, ... arguments of the reference's kernel layers, parameters/StandardParameters.hpp:61-76; 0 = none),
	 * enforced where StandardParameters enforces them (:105-123, :150-182).
	 */
	inline void set_constraints(std::size_t index, Scalar value_clip, Scalar value_max_l1_norm, Scalar value_max_l2_norm,
			Scalar grad_clip, Scalar grad_max_l1_norm, Scalar grad_max_l2_norm) {
		check(cattle_hip_layer_param_set_constraints(handle, index, (double) value_clip, (double) value_max_l1_norm,
				(double) value_max_l2_norm, (double) grad_clip, (double) grad_max_l1_norm, (double) grad_max_l2_norm));
	}
	/** The sum of Parameters::get_regularization_penalty over the layer's parameters (optimizer/SGDOptimizer.hpp:62). */
	inline Scalar get_regularization_penalty() const {
		const std::size_t n = num_params();
		double total = 0, one = 0;
		for (std::size_t i = 0; i < n; ++i) {
			check(cattle_hip_layer_param_regularization_penalty(handle, i, &one));
			total += one;
		}
		return (Scalar) total;
	}
	/** reset_grad of every parameter (optimizer/SGDOptimizer.hpp:68-70). */
	inline void reset_grads() {
		const std::size_t n = num_params();
		for (std::size_t i = 0; i < n; ++i)
			check(cattle_hip_layer_reset_param_grad(handle, i));
	}
	/** VanillaSGDOptimizer::_update_params over this layer's optimizable parameters. */
	inline void sgd_update(Scalar learning_rate) {
		for_each_optimizable([&](std::size_t i) {
			check(cattle_hip_layer_param_sgd_update(handle, i, (double) learning_rate));
		});
	}
	/** AdamOptimizer::_update_params over this layer's optimizable parameters (defaults of AdamOptimizer.hpp:40-42). */
	inline void adam_update(std::size_t timestep, Scalar learning_rate = 1e-3, Scalar l1_decay = 1e-1,
			Scalar l2_decay = 1e-3, Scalar epsilon = 1e-5) {
		for_each_optimizable([&](std::size_t i) {
			check(cattle_hip_layer_param_adam_update(handle, i, (double) learning_rate, (double) l1_decay, (double) l2_decay,
					(double) epsilon, timestep));
		});
	}
	/**
	 * The update of every optimizable parameter followed by its reset_grad, as SGDOptimizer::_train applies them to
	 * a batch (optimizer/SGDOptimizer.hpp:64, :68-70); the gradient is zeroed by the update kernel itself. Gradients
	 * of non-optimizable parameters are never accumulated (parameters/StandardParameters.hpp:116-117) and stay zero.
	 */
	inline void optimizer_step(cattle_hip_optimizer optimizer, const double (&hyper)[4], std::size_t epoch, std::size_t timestep) {
		for_each_optimizable([&](std::size_t i) {
			check(cattle_hip_layer_param_optimizer_step(handle, i, optimizer, hyper, epoch, timestep));
		});
	}
	/** Appends (handle, index) of every optimizable parameter of this layer. */
	inline void append_optimizable(std::vector<cattle_hip_layer_t>& handles, std::vector<std::size_t>& indices) {
		for_each_optimizable([&](std::size_t i) {
			handles.push_back(handle);
			indices.push_back(i);
		});
	}
	/** AdamOptimizer::_fit. */
	inline void reset_optimizer_state() {
		const std::size_t n = num_params();
		for (std::size_t i = 0; i < n; ++i)
			check(cattle_hip_layer_param_reset_optimizer_state(handle, i));
	}
	inline cattle_hip_layer_t get() const {
		return handle;
	}
	/**
	 * The layer's parameter matrices the way the reference layer's get_params() lists them: a per-channel batch
	 * norm holds four 1x1 matrices per channel (layer/BatchNormLayer.hpp:263-272) where the device holds four
	 * 1 x channels rows; every other layer's lists coincide. Each entry is (rows, cols, values).
	 */
	struct HostMatrix {
		std::size_t rows, cols;
		std::vector<Scalar> values;
	};
	inline std::vector<HostMatrix> get_reference_params() const {
		std::vector<HostMatrix> out;
		const std::size_t n = num_params();
		if (!params_per_column) {
			for (std::size_t i = 0; i < n; ++i) {
				HostMatrix m;
				bool opt;
				param_shape(i, m.rows, m.cols, opt);
				m.values = get_param_values(i);
				out.push_back(std::move(m));
			}
			return out;
		}
		std::vector<std::vector<Scalar>> rows(n);
		for (std::size_t i = 0; i < n; ++i)
			rows[i] = get_param_values(i);
		for (std::size_t c = 0; c < rows[0].size(); ++c)
			for (std::size_t i = 0; i < n; ++i)
				out.push_back(HostMatrix{ 1, 1, std::vector<Scalar>(1, rows[i][c]) });
		return out;
	}
	/** The inverse of get_reference_params(): consumes this layer's matrices from `mats` starting at `pos`. */
	inline void set_reference_params(const std::vector<HostMatrix>& mats, std::size_t& pos) {
		const std::size_t n = num_params();
		for (std::size_t i = 0; i < n; ++i) {
			std::size_t rows, cols;
			bool opt;
			param_shape(i, rows, cols, opt);
			if (!params_per_column) {
				if (pos >= mats.size() || mats[pos].rows != rows || mats[pos].cols != cols)
					throw std::runtime_error("parameter matrix of unexpected dimensions");
				set_param_values(i, mats[pos++].values.data());
			}
		}
		if (params_per_column && n > 0) {
			std::size_t rows, cols;
			bool opt;
			param_shape(0, rows, cols, opt);
			if (pos + n * cols > mats.size())
				throw std::runtime_error("too few parameter matrices");
			std::vector<std::vector<Scalar>> vals(n, std::vector<Scalar>(cols));
			for (std::size_t c = 0; c < cols; ++c)
				for (std::size_t i = 0; i < n; ++i) {
					const HostMatrix& m = mats[pos++];
					if (m.rows != 1 || m.cols != 1)
						throw std::runtime_error("parameter matrix of unexpected dimensions");
					vals[i][c] = m.values[0];
				}
			for (std::size_t i = 0; i < n; ++i)
				set_param_values(i, vals[i].data());
			if (n == 4)       /* running statistics were loaded: the layer may infer (BatchNormLayer.hpp:234-243) */
				check(cattle_hip_batchnorm_set_stats_initialized(handle, 1));
		}
	}
private:
	inline explicit DeviceLayer(cattle_hip_layer_t handle) : handle(handle), params_per_column(false), kernel_layer(false) {
		std::size_t d[3];
		check(cattle_hip_layer_input_dims(handle, d));
		in_dims = Dims{ { d[0], d[1], d[2] } };
		check(cattle_hip_layer_output_dims(handle, d));
		out_dims = Dims{ { d[0], d[1], d[2] } };
	}
	/* dense and activation layers are created from a volume: keep the caller's shape for the tensors */
	inline DeviceLayer(cattle_hip_layer_t handle, const Dims& in) : DeviceLayer(handle) {
		in_dims = in;
	}
	inline DeviceLayer(cattle_hip_layer_t handle, const Dims& in, const Dims& out) : handle(handle), in_dims(in),
			out_dims(out), params_per_column(false), kernel_layer(false) { }
	template<typename Fn>
	inline void for_each_optimizable(Fn fn) {
		const std::size_t n = num_params();
		for (std::size_t i = 0; i < n; ++i) {
			std::size_t rows, cols;
			bool optimizable;
			param_shape(i, rows, cols, optimizable);
			if (optimizable)
				fn(i);
		}
	}
	inline std::vector<Scalar> fetch(std::size_t index, int (*getter)(cattle_hip_layer_t, size_t, void*, cattle_hip_memspace)) const {
		std::size_t rows, cols;
		bool optimizable;
		param_shape(index, rows, cols, optimizable);
		std::vector<Scalar> out(rows * cols);
		check(getter(handle, index, out.data(), CATTLE_HIP_HOST));
		return out;
	}
	cattle_hip_layer_t handle;
	Dims in_dims, out_dims;
	DeviceTensor<Scalar> cached_in, cached_out;
	bool params_per_column;
	bool kernel_layer;          /* a weight matrix (parameter 0) and a bias (parameter 1): conv, transposed conv, dense */
};

/**
 * Loss::function / d_function on device tensors (loss/UniversalLoss.hpp:27-55, non-sequential data) for every
 * loss of the loss/ directory; `negated` wraps it as NegatedLoss does (loss/NegatedLoss.hpp:41-46).
 */
template<typename Scalar>
class DeviceLoss {
public:
	inline explicit DeviceLoss(cattle_hip_loss kind, Scalar epsilon = 1e-5, bool negated = false) :
			kind((cattle_hip_loss) (negated ? kind | CATTLE_HIP_LOSS_NEGATED : kind)), epsilon(epsilon) { }
	/** The per-sample losses, on the host (a column vector in the reference). */
	inline std::vector<Scalar> function(const DeviceTensor<Scalar>& out, const DeviceTensor<Scalar>& obj) const {
		assert(out.dimensions() == obj.dimensions());
		std::vector<Scalar> losses(out.batch());
		check(cattle_hip_loss_function(Code<Scalar>::value, kind, out.data(), CATTLE_HIP_DEVICE, obj.data(),
				CATTLE_HIP_DEVICE, out.batch(), 1, out.size() / out.batch(), (double) epsilon, losses.data(),
				CATTLE_HIP_HOST));
		return losses;
	}
	/** scale * d_function; scale = 1 / batch_size is the optimizer's division (optimizer/SGDOptimizer.hpp:54-55). */
	/** The same values left on the device: `losses` holds one scalar per sample (dims { batch, 1, 1, 1 }). */
	inline void function_into(const DeviceTensor<Scalar>& out, const DeviceTensor<Scalar>& obj, DeviceTensor<Scalar>& losses) const {
		assert(out.dimensions() == obj.dimensions() && losses.size() == out.batch());
		check(cattle_hip_loss_function(Code<Scalar>::value, kind, out.data(), CATTLE_HIP_DEVICE, obj.data(), CATTLE_HIP_DEVICE,
				out.batch(), 1, out.size() / out.batch(), (double) epsilon, losses.data(), CATTLE_HIP_DEVICE));
	}
	inline DeviceTensor<Scalar> d_function(const DeviceTensor<Scalar>& out, const DeviceTensor<Scalar>& obj,
			Scalar scale = 1) const {
		assert(out.dimensions() == obj.dimensions());
		DeviceTensor<Scalar> grad(out.dimensions());
		check(cattle_hip_loss_d_function(Code<Scalar>::value, kind, out.data(), CATTLE_HIP_DEVICE, obj.data(),
				CATTLE_HIP_DEVICE, out.batch(), 1, out.size() / out.batch(), (double) epsilon, (double) scale, grad.data(),
				CATTLE_HIP_DEVICE));
		return grad;
	}
private:
	cattle_hip_loss kind;
	Scalar epsilon;
};

/**
 * A recorded sequence of device-side calls (cattle_hip_graph_*): what is issued between begin() and end() is recorded
 * instead of run, and launch() runs it as one HIP graph. The calls must have run once before, must use device tensors
 * only and must read nothing back; tensors that were created during the recording stay allocated until the graph goes.
 */
class DeviceGraph {
public:
	inline DeviceGraph() : handle(nullptr) { }
	DeviceGraph(const DeviceGraph&) = delete;
	DeviceGraph& operator=(const DeviceGraph&) = delete;
	inline DeviceGraph(DeviceGraph&& other) : handle(other.handle) {
		other.handle = nullptr;
	}
	inline ~DeviceGraph() {
		if (handle)
			cattle_hip_graph_destroy(handle);
	}
	inline void begin() {
		check(cattle_hip_graph_begin_capture());
	}
	inline void end() {
		check(cattle_hip_graph_end_capture(&handle));
	}
	inline void launch() const {
		check(cattle_hip_graph_launch(handle));
	}
	inline bool is_recorded() const {
		return handle != nullptr;
	}
private:
	cattle_hip_graph_t handle;
};

/**
 * A stack of device layers (neural_network/FeedforwardNeuralNetwork.hpp:38-53, :112-127 on device
 * tensors): layer 0 is the input layer when the network is foremost.
 */
template<typename Scalar>
class DeviceFeedforwardNetwork {
public:
	inline explicit DeviceFeedforwardNetwork(std::vector<DeviceLayer<Scalar>> layers, bool foremost = true) :
			layers(std::move(layers)),
			foremost(foremost),
			frozen(false) {
		assert(!this->layers.empty());
		this->layers[0].set_input_layer(foremost);
		for (std::size_t i = 0; i < this->layers.size(); ++i)
			units.push_back(Unit{ i, 1, NO_FUSED });
	}
	inline std::vector<DeviceLayer<Scalar>>& get_layers() {
		return layers;
	}
	/**
	 * From now on every kernel layer and the batch norm, element-wise activation and pool layers right behind it run as one
	 * fused layer (DeviceLayer::fused): the same calls as FeedforwardNeuralNetwork.hpp:112-141 makes, with the activation,
	 * the max pooling and the batch-norm moments computed in the epilogue of the layer's GEMM. get_layers(), the
	 * parameters and everything that works on them are unaffected. Returns the number of fused groups.
	 */
	inline std::size_t fuse() {
		units.clear();
		fused_layers.clear();
		std::size_t i = 0;
		while (i < layers.size()) {
			std::size_t len = 1;
			if (layers[i].is_kernel_layer()) {
				for (len = layers.size() - i < 4 ? layers.size() - i : 4; len > 1; --len) {
					const DeviceLayer<Scalar>* members[4];
					for (std::size_t k = 0; k < len; ++k)
						members[k] = &layers[i + k];
					DeviceLayer<Scalar> f = DeviceLayer<Scalar>::fused(members, len);
					if (!f.is_null()) {
						fused_layers.push_back(std::move(f));
						break;
					}
				}
			}
			units.push_back(Unit{ i, len, len > 1 ? fused_layers.size() - 1 : NO_FUSED });
			i += len;
		}
		if (units[0].fused != NO_FUSED)
			fused_layers[units[0].fused].set_input_layer(foremost);
		return fused_layers.size();
	}
	inline const typename DeviceLayer<Scalar>::Dims& get_input_dims() const {
		return layers.front().get_input_dims();
	}
	inline const typename DeviceLayer<Scalar>::Dims& get_output_dims() const {
		return layers.back().get_output_dims();
	}
	/** neural_network/FeedforwardNeuralNetwork.hpp:88-94 */
	inline bool is_foremost() const {
		return foremost;
	}
	inline void set_foremost(bool foremost) {
		layers[0].set_input_layer(foremost);
		if (units[0].fused != NO_FUSED)
			fused_layers[units[0].fused].set_input_layer(foremost);
		this->foremost = foremost;
	}
	/**
	 * NeuralNetwork::set_frozen (core/NeuralNetwork.hpp:166-169): the parameters of a frozen network still receive
	 * gradients, optimizers leave their values alone and reset the gradients (optimizer/SGDOptimizer.hpp:58-70).
	 */
	inline bool is_frozen() const {
		return frozen;
	}
	inline void set_frozen(bool frozen) {
		this->frozen = frozen;
	}
	/** NeuralNetwork::infer (core/NeuralNetwork.hpp:225-228); the result lives until the next pass of the network. */
	inline const DeviceTensor<Scalar>& infer(const DeviceTensor<Scalar>& input) {
		return propagate(input, false);
	}
	inline void reset_grads() {
		for (std::size_t i = 0; i < layers.size(); ++i)
			layers[i].reset_grads();
	}
	/**
	 * NeuralNetwork::init (core/NeuralNetwork.hpp:173-176) with one weight initialization for all kernel layers: the
	 * weight matrices (parameter 0 of the layers that have a weight matrix and a bias) take `weight_init`; biases,
	 * batch-norm and activation parameters are back at the values their layers are created with (zero biases,
	 * gamma 1 / beta 0, the constant of PReLU and PSwish), which is what the reference's layers initialize them to.
	 */
	inline void init(const ParameterInitialization<Scalar>& weight_init) {
		for (std::size_t l = 0; l < layers.size(); ++l) {
			if (!layers[l].is_kernel_layer())
				continue;
			layers[l].init_params(0, weight_init);
			layers[l].init_params(1, ConstantParameterInitialization<Scalar>(0));
		}
	}
	/** The regularization loss SGDOptimizer::_train reports beside the objective (optimizer/SGDOptimizer.hpp:59-63). */
	inline Scalar get_regularization_penalty() const {
		Scalar total = 0;
		for (std::size_t i = 0; i < layers.size(); ++i)
			total += layers[i].get_regularization_penalty();
		return total;
	}
	/**
	 * NeuralNetwork::save_all_unique_params_values / load_all_unique_params_values in the binary format
	 * (core/NeuralNetwork.hpp:195-223): one file <dir>/<prefix><i>.prms per parameter matrix in get_params() order,
	 * each an unsigned short scalar size, unsigned rows, unsigned cols and the column-major coefficients
	 * (core/EigenProxy.hpp:147-159, :212-224), so that networks trained by either side resume on the other.
	 */
	inline void save_all_unique_params_values(const std::string& dir_path,
			const std::string& file_name_prefix = "c-attl3_neural_net_params_") const {
		std::size_t index = 0;
		for (std::size_t l = 0; l < layers.size(); ++l) {
			const std::vector<typename DeviceLayer<Scalar>::HostMatrix> mats = layers[l].get_reference_params();
			for (std::size_t i = 0; i < mats.size(); ++i) {
				std::ofstream out(dir_path + "/" + file_name_prefix + std::to_string(index++) + ".prms", std::ios::binary);
				if (!out.is_open())
					throw std::runtime_error("cannot write a parameter file under " + dir_path);
				const unsigned short scalar_size = (unsigned short) sizeof(Scalar);
				const unsigned rows = (unsigned) mats[i].rows, cols = (unsigned) mats[i].cols;
				out.write(reinterpret_cast<const char*>(&scalar_size), sizeof(scalar_size));
				out.write(reinterpret_cast<const char*>(&rows), sizeof(rows));
				out.write(reinterpret_cast<const char*>(&cols), sizeof(cols));
				out.write(reinterpret_cast<const char*>(mats[i].values.data()), (std::streamsize) (mats[i].values.size() * sizeof(Scalar)));
			}
		}
	}
	inline void load_all_unique_params_values(const std::string& dir_path,
			const std::string& file_name_prefix = "c-attl3_neural_net_params_") {
		std::vector<typename DeviceLayer<Scalar>::HostMatrix> mats;
		for (;;) {
			std::ifstream in(dir_path + "/" + file_name_prefix + std::to_string(mats.size()) + ".prms", std::ios::binary);
			if (!in.is_open())
				break;
			unsigned short scalar_size = 0;
			unsigned rows = 0, cols = 0;
			in.read(reinterpret_cast<char*>(&scalar_size), sizeof(scalar_size));
			in.read(reinterpret_cast<char*>(&rows), sizeof(rows));
			in.read(reinterpret_cast<char*>(&cols), sizeof(cols));
			if (!in || scalar_size != sizeof(Scalar))          /* assert(scalar_size == sizeof(Scalar)) */
				throw std::runtime_error("parameter file of another scalar type or truncated");
			typename DeviceLayer<Scalar>::HostMatrix m;
			m.rows = rows;
			m.cols = cols;
			m.values.resize((std::size_t) rows * cols);
			in.read(reinterpret_cast<char*>(m.values.data()), (std::streamsize) (m.values.size() * sizeof(Scalar)));
			if (!in)
				throw std::runtime_error("truncated parameter file");
			mats.push_back(std::move(m));
		}
		std::size_t pos = 0;
		for (std::size_t l = 0; l < layers.size(); ++l)
			layers[l].set_reference_params(mats, pos);
		if (pos != mats.size())
			throw std::runtime_error("more parameter files than the network has parameters");
	}
	/** propagate: `input` must stay alive and unmodified until backpropagate returns. */
	inline const DeviceTensor<Scalar>& propagate(const DeviceTensor<Scalar>& input, bool training) {
		const DeviceTensor<Scalar>* cur = &unit(0).pass_forward_borrowed(input, training);
		for (std::size_t i = 1; i < units.size(); ++i)
			cur = &unit(i).pass_forward_borrowed(*cur, training);        /* the producer keeps its output alive */
		return *cur;
	}
	inline DeviceTensor<Scalar> backpropagate(const DeviceTensor<Scalar>& out_grad) {
		DeviceTensor<Scalar> grad;
		for (std::size_t i = units.size(); i-- > 0;) {
			const bool needs = !(i == 0 && foremost);
			grad = unit(i).pass_back(i + 1 == units.size() ? out_grad : grad, needs);
		}
		return grad;
	}
	/**
	 * One batch of SGDOptimizer::_train (optimizer/SGDOptimizer.hpp:44-70) with the vanilla SGD or the
	 * Adam update: propagate, loss, gradient / batch size, backpropagate, update, reset. Returns the
	 * sum of the per-sample losses of the batch.
	 */
	/** The same with any of the optimizers; `hyper` holds the optimizer's constructor arguments (include/cattle_hip.h). */
	inline Scalar train_batch(const DeviceTensor<Scalar>& input, const DeviceTensor<Scalar>& obj, const DeviceLoss<Scalar>& loss,
			cattle_hip_optimizer optimizer, const double (&hyper)[4], std::size_t epoch, std::size_t timestep) {
		const Scalar total = forward_backward(input, obj, loss);
		optimizer_step(optimizer, hyper, epoch, timestep);
		return total;
	}
	inline Scalar train_batch_sgd(const DeviceTensor<Scalar>& input, const DeviceTensor<Scalar>& obj,
			const DeviceLoss<Scalar>& loss, Scalar learning_rate) {
		const Scalar total = forward_backward(input, obj, loss);
		const double hyper[4] = { (double) learning_rate, 0, 0, 0 };
		optimizer_step(CATTLE_HIP_OPT_VANILLA_SGD, hyper, 0, 0);
		return total;
	}
	inline Scalar train_batch_adam(const DeviceTensor<Scalar>& input, const DeviceTensor<Scalar>& obj,
			const DeviceLoss<Scalar>& loss, std::size_t timestep, Scalar learning_rate = 1e-3, Scalar l1_decay = 1e-1,
			Scalar l2_decay = 1e-3, Scalar epsilon = 1e-5) {
		const Scalar total = forward_backward(input, obj, loss);
		const double hyper[4] = { (double) learning_rate, (double) l1_decay, (double) l2_decay, (double) epsilon };
		optimizer_step(CATTLE_HIP_OPT_ADAM, hyper, 0, timestep);
		return total;
	}
	/**
	 * One batch of SGDOptimizer::_train on fixed tensors, recorded once and repeated by every run(): propagate, the loss
	 * of every sample, its gradient / batch size, backpropagate as one graph launch, then the optimizer step (outside the
	 * graph: its scalars, the time step for one, change from batch to batch) and the read-back of the losses. The caller
	 * refills `input` and `obj` in place between runs. Call train_batch once on the same tensors first, so that every
	 * buffer of the layers exists when the recording starts.
	 */
	class RecordedBatch {
	public:
		inline Scalar run(cattle_hip_optimizer optimizer, const double (&hyper)[4], std::size_t epoch, std::size_t timestep) {
			graph.launch();
			net->optimizer_step(optimizer, hyper, epoch, timestep);
			const std::vector<Scalar> host = losses.to_host();
			Scalar total = 0;
			for (std::size_t i = 0; i < host.size(); ++i)
				total += host[i];
			return total;
		}
	private:
		friend class DeviceFeedforwardNetwork;
		inline RecordedBatch(DeviceFeedforwardNetwork* net, std::size_t batch) : net(net),
				losses(typename DeviceTensor<Scalar>::Dims{ { batch, 1, 1, 1 } }) { }
		DeviceFeedforwardNetwork* net;
		DeviceTensor<Scalar> losses;
		DeviceGraph graph;
	};
	inline RecordedBatch record_batch(const DeviceTensor<Scalar>& input, const DeviceTensor<Scalar>& obj, const DeviceLoss<Scalar>& loss) {
		RecordedBatch rec(this, input.batch());
		rec.graph.begin();
		try {
			const DeviceTensor<Scalar>& out = propagate(input, true);
			loss.function_into(out, obj, rec.losses);
			backpropagate(loss.d_function(out, obj, (Scalar) 1 / (Scalar) input.batch()));
		} catch (...) {
			cattle_hip_graph_t dropped = nullptr;
			if (cattle_hip_graph_end_capture(&dropped) == CATTLE_HIP_OK)
				cattle_hip_graph_destroy(dropped);
			throw;
		}
		rec.graph.end();
		return rec;
	}
	/**
	 * The update of every optimizable parameter of the network followed by its reset_grad
	 * (optimizer/SGDOptimizer.hpp:64, :68-70), sixteen parameters per launch.
	 */
	inline void optimizer_step(cattle_hip_optimizer optimizer, const double (&hyper)[4], std::size_t epoch, std::size_t timestep) {
		if (frozen) {
			reset_grads();
			return;
		}
		std::vector<cattle_hip_layer_t> handles;
		std::vector<std::size_t> indices;
		for (std::size_t i = 0; i < layers.size(); ++i)
			layers[i].append_optimizable(handles, indices);
		if (!handles.empty())
			check(cattle_hip_optimizer_step_many(handles.data(), indices.data(), handles.size(), optimizer, hyper, epoch, timestep));
	}
private:
	inline Scalar forward_backward(const DeviceTensor<Scalar>& input, const DeviceTensor<Scalar>& obj,
			const DeviceLoss<Scalar>& loss) {
		const DeviceTensor<Scalar>& out = propagate(input, true);
		const std::vector<Scalar> losses = loss.function(out, obj);
		Scalar total = 0;
		for (std::size_t i = 0; i < losses.size(); ++i)
			total += losses[i];
		backpropagate(loss.d_function(out, obj, (Scalar) 1 / (Scalar) input.batch()));
		return total;
	}
	/* what propagate calls: one layer, or `count` layers from `first` on through the fused layer over them */
	struct Unit {
		std::size_t first, count, fused;
	};
	static constexpr std::size_t NO_FUSED = (std::size_t) -1;
	inline DeviceLayer<Scalar>& unit(std::size_t i) {
		return units[i].fused == NO_FUSED ? layers[units[i].first] : fused_layers[units[i].fused];
	}
	std::vector<DeviceLayer<Scalar>> layers;
	std::vector<DeviceLayer<Scalar>> fused_layers;      /* declared after `layers`: destroyed before the members they borrow */
	std::vector<Unit> units;
	bool foremost, frozen;
};

template<typename Scalar>
constexpr std::size_t DeviceFeedforwardNetwork<Scalar>::NO_FUSED;

/**
 * Feed-forward networks on top of one another (neural_network/StackedNeuralNetwork.hpp:33-120 on device tensors): only
 * the first module can be foremost; propagate and backpropagate run through the modules in order and in reverse. Each
 * module keeps its own frozen flag, so one optimizer step can update some modules and only reset the gradients of others,
 * as the reference's generative-adversarial example does (examples/mnist_gan.cpp:107-109).
 */
template<typename Scalar>
class DeviceStackedNetwork {
public:
	typedef DeviceFeedforwardNetwork<Scalar> Module;
	inline explicit DeviceStackedNetwork(std::vector<Module> modules, bool foremost = true) : modules(std::move(modules)) {
		if (this->modules.empty())
			throw std::invalid_argument("modules must contain at least 1 element");
		for (std::size_t i = 1; i < this->modules.size(); ++i) {
			if (this->modules[i - 1].get_output_dims() != this->modules[i].get_input_dims())
				throw std::invalid_argument("incompatible network dimensions");
			this->modules[i].set_foremost(false);
		}
		this->modules[0].set_foremost(foremost);
	}
	inline std::vector<Module>& get_modules() {
		return modules;
	}
	inline bool is_foremost() const {
		return modules[0].is_foremost();
	}
	inline void set_foremost(bool foremost) {
		modules[0].set_foremost(foremost);
	}
	inline void set_frozen(bool frozen) {
		for (std::size_t i = 0; i < modules.size(); ++i)
			modules[i].set_frozen(frozen);
	}
	/** `input` must stay alive and unmodified until backpropagate returns. */
	inline const DeviceTensor<Scalar>& propagate(const DeviceTensor<Scalar>& input, bool training) {
		const DeviceTensor<Scalar>* cur = &modules[0].propagate(input, training);
		for (std::size_t i = 1; i < modules.size(); ++i)
			cur = &modules[i].propagate(*cur, training);
		return *cur;
	}
	inline const DeviceTensor<Scalar>& infer(const DeviceTensor<Scalar>& input) {
		return propagate(input, false);
	}
	inline DeviceTensor<Scalar> backpropagate(const DeviceTensor<Scalar>& out_grad) {
		DeviceTensor<Scalar> grad = modules.back().backpropagate(out_grad);
		for (std::size_t i = modules.size() - 1; i-- > 0;)
			grad = modules[i].backpropagate(grad);
		return grad;
	}
	inline void optimizer_step(cattle_hip_optimizer optimizer, const double (&hyper)[4], std::size_t epoch, std::size_t timestep) {
		for (std::size_t i = 0; i < modules.size(); ++i)
			modules[i].optimizer_step(optimizer, hyper, epoch, timestep);
	}
	/** One batch of SGDOptimizer::_train (optimizer/SGDOptimizer.hpp:44-70); returns the sum of the per-sample losses. */
	inline Scalar train_batch(const DeviceTensor<Scalar>& input, const DeviceTensor<Scalar>& obj, const DeviceLoss<Scalar>& loss,
			cattle_hip_optimizer optimizer, const double (&hyper)[4], std::size_t epoch, std::size_t timestep) {
		const DeviceTensor<Scalar>& out = propagate(input, true);
		const std::vector<Scalar> losses = loss.function(out, obj);
		Scalar total = 0;
		for (std::size_t i = 0; i < losses.size(); ++i)
			total += losses[i];
		backpropagate(loss.d_function(out, obj, (Scalar) 1 / (Scalar) input.batch()));
		optimizer_step(optimizer, hyper, epoch, timestep);
		return total;
	}
private:
	std::vector<Module> modules;
};

/**
 * LSTMNeuralNetwork<Scalar,3> over eight ConvKernelLayers with fused gates, on device tensors
 * (neural_network/LSTMNeuralNetwork.hpp:27-120, :236-503; multiplicative integration by
 * set_multiplicative_integration; not stateful, not reversed). An LSTM over vectors, with DenseKernelLayers, is the case
 * of 1 x 1 images and 1 x 1 receptors without padding. Sequences are (batch, time, height, width, channels) column-major.
 */
template<typename Scalar>
class DeviceConvLSTM {
public:
	typedef std::array<std::size_t,3> Dims;
	/** (output sequence length, output delay) for an input sequence length: the OutputSeqSizeFunc (:60-63). */
	typedef std::pair<std::size_t,std::size_t> (*OutputSeqSizeFunc)(std::size_t);
	/** A sequence on the device: dims (batch, time, height, width, channels). */
	struct Sequence {
		std::array<std::size_t,5> dims;
		DeviceTensor<Scalar> data;       /* stored as (batch * time, height, width, channels) */
	};
	/* kernels in the order of get_layers() (:521-529) */
	enum Kernel { INPUT_FORGET = 0, OUTPUT_FORGET, INPUT_WRITE, OUTPUT_WRITE, INPUT_CANDIDATE, OUTPUT_CANDIDATE, INPUT_READ,
		OUTPUT_READ };
	inline DeviceConvLSTM(const Dims& input_dims, std::size_t hidden_channels, OutputSeqSizeFunc output_seq_size_func,
			bool foremost = true, std::size_t receptor_height = 3, std::size_t receptor_width = 3,
			std::size_t vertical_padding = 1, std::size_t horizontal_padding = 1, std::size_t vertical_dilation = 0,
			std::size_t horizontal_dilation = 0, cattle_hip_activation forget_act = CATTLE_HIP_ACT_SIGMOID,
			cattle_hip_activation write_act = CATTLE_HIP_ACT_SIGMOID, cattle_hip_activation candidate_act = CATTLE_HIP_ACT_TANH,
			cattle_hip_activation state_act = CATTLE_HIP_ACT_TANH, cattle_hip_activation read_act = CATTLE_HIP_ACT_SIGMOID) :
				handle(nullptr), input_dims(input_dims), hidden(hidden_channels), seq(output_seq_size_func), foremost(foremost),
				batch(0), in_len(0) {
		const int kinds[5] = { forget_act, write_act, candidate_act, state_act, read_act };
		check(cattle_hip_convlstm_create(Code<Scalar>::value, input_dims[0], input_dims[1], input_dims[2], hidden_channels,
				receptor_height, receptor_width, vertical_padding, horizontal_padding, vertical_dilation, horizontal_dilation,
				kinds, nullptr, foremost ? 1 : 0, &handle));
	}
	DeviceConvLSTM(const DeviceConvLSTM&) = delete;
	DeviceConvLSTM& operator=(const DeviceConvLSTM&) = delete;
	inline ~DeviceConvLSTM() {
		if (handle)
			cattle_hip_layer_destroy(handle);
	}
	/** The MulInt template argument of the reference network (neural_network/LSTMNeuralNetwork.hpp:44, :303-311). */
	inline void set_multiplicative_integration(bool enabled) {
		check(cattle_hip_convlstm_set_multiplicative_integration(handle, enabled ? 1 : 0));
	}
	inline void set_kernel_values(Kernel kernel, bool bias, const Scalar* host_values) {
		check(cattle_hip_convlstm_set_kernel_values(handle, (std::size_t) kernel, bias ? 1 : 0, host_values, CATTLE_HIP_HOST));
	}
	inline std::vector<Scalar> get_kernel_values(Kernel kernel, bool bias) const {
		std::vector<Scalar> out(kernel_size(kernel, bias));
		check(cattle_hip_convlstm_get_kernel_values(handle, (std::size_t) kernel, bias ? 1 : 0, out.data(), CATTLE_HIP_HOST));
		return out;
	}
	inline std::vector<Scalar> get_kernel_grad(Kernel kernel, bool bias) const {
		std::vector<Scalar> out(kernel_size(kernel, bias));
		check(cattle_hip_convlstm_get_kernel_grad(handle, (std::size_t) kernel, bias ? 1 : 0, out.data(), CATTLE_HIP_HOST));
		return out;
	}
	/** Rows of a kernel's weight matrix times hidden_channels, or hidden_channels for a bias. */
	inline std::size_t kernel_size(Kernel kernel, bool bias) const {
		std::size_t rows, cols;
		int opt;
		check(cattle_hip_layer_param_shape(handle, ((std::size_t) kernel % 2) * 2, &rows, &cols, &opt));
		return bias ? hidden : rows * hidden;
	}
	/**
	 * NeuralNetwork::save_all_unique_params_values / load_all_unique_params_values (core/NeuralNetwork.hpp:195-223) for
	 * the LSTM: the parameter matrices in get_layers() order (:521-534), i.e. weights then bias of the eight kernels
	 * (the five activations have none), each in the binary format of core/EigenProxy.hpp:147-159, :212-224.
	 */
	inline void save_all_unique_params_values(const std::string& dir_path,
			const std::string& file_name_prefix = "c-attl3_neural_net_params_") const {
		for (std::size_t i = 0; i < 16; ++i) {
			const Kernel kernel = (Kernel) (i / 2);
			const bool bias = i % 2 == 1;
			const std::vector<Scalar> values = get_kernel_values(kernel, bias);
			std::ofstream out(dir_path + "/" + file_name_prefix + std::to_string(i) + ".prms", std::ios::binary);
			if (!out.is_open())
				throw std::runtime_error("cannot write a parameter file under " + dir_path);
			const unsigned short scalar_size = (unsigned short) sizeof(Scalar);
			const unsigned rows = bias ? 1u : (unsigned) (values.size() / hidden), cols = (unsigned) hidden;
			out.write(reinterpret_cast<const char*>(&scalar_size), sizeof(scalar_size));
			out.write(reinterpret_cast<const char*>(&rows), sizeof(rows));
			out.write(reinterpret_cast<const char*>(&cols), sizeof(cols));
			out.write(reinterpret_cast<const char*>(values.data()), (std::streamsize) (values.size() * sizeof(Scalar)));
		}
	}
	inline void load_all_unique_params_values(const std::string& dir_path,
			const std::string& file_name_prefix = "c-attl3_neural_net_params_") {
		for (std::size_t i = 0; i < 16; ++i) {
			const Kernel kernel = (Kernel) (i / 2);
			const bool bias = i % 2 == 1;
			std::ifstream in(dir_path + "/" + file_name_prefix + std::to_string(i) + ".prms", std::ios::binary);
			if (!in.is_open())
				throw std::runtime_error("missing parameter file " + std::to_string(i) + " under " + dir_path);
			unsigned short scalar_size = 0;
			unsigned rows = 0, cols = 0;
			in.read(reinterpret_cast<char*>(&scalar_size), sizeof(scalar_size));
			in.read(reinterpret_cast<char*>(&rows), sizeof(rows));
			in.read(reinterpret_cast<char*>(&cols), sizeof(cols));
			if (!in || scalar_size != sizeof(Scalar))          /* assert(scalar_size == sizeof(Scalar)) */
				throw std::runtime_error("parameter file of another scalar type or truncated");
			if ((std::size_t) rows * cols != kernel_size(kernel, bias) || cols != hidden)
				throw std::runtime_error("parameter file " + std::to_string(i) + " does not have the kernel's dimensions");
			std::vector<Scalar> values((std::size_t) rows * cols);
			in.read(reinterpret_cast<char*>(values.data()), (std::streamsize) (values.size() * sizeof(Scalar)));
			if (!in)
				throw std::runtime_error("truncated parameter file");
			set_kernel_values(kernel, bias, values.data());
		}
	}
	/** propagate (:236-403): `input` must stay alive and unmodified until backpropagate returns. */
	inline Sequence propagate(const Sequence& input, bool training) {
		const std::pair<std::size_t,std::size_t> out_seq = seq(input.dims[1]);
		Sequence out;
		out.dims = { { input.dims[0], out_seq.first, input_dims[0], input_dims[1], hidden } };
		out.data = DeviceTensor<Scalar>(typename DeviceTensor<Scalar>::Dims{ { input.dims[0] * out_seq.first, input_dims[0],
				input_dims[1], hidden } });
		check(cattle_hip_convlstm_propagate(handle, input.data.data(), CATTLE_HIP_DEVICE, input.dims[0], input.dims[1],
				out_seq.first, out_seq.second, training ? 1 : 0, out.data.data(), CATTLE_HIP_DEVICE));
		batch = input.dims[0];
		in_len = input.dims[1];
		return out;
	}
	/** backpropagate (:404-503): the input gradient, with a null tensor when the network is foremost. */
	inline Sequence backpropagate(const Sequence& out_grad) {
		Sequence grad;
		grad.dims = { { batch, in_len, input_dims[0], input_dims[1], input_dims[2] } };
		if (!foremost)
			grad.data = DeviceTensor<Scalar>(typename DeviceTensor<Scalar>::Dims{ { batch * in_len, input_dims[0],
					input_dims[1], input_dims[2] } });
		check(cattle_hip_convlstm_backpropagate(handle, out_grad.data.data(), CATTLE_HIP_DEVICE,
				foremost ? nullptr : grad.data.data(), CATTLE_HIP_DEVICE));
		return grad;
	}
	/** Optimizer updates and gradient reset over the four fused parameters. */
	inline void sgd_update(Scalar learning_rate) {
		for (std::size_t i = 0; i < 4; ++i)
			check(cattle_hip_layer_param_sgd_update(handle, i, (double) learning_rate));
	}
	inline void adam_update(std::size_t timestep, Scalar learning_rate = 1e-3, Scalar l1_decay = 1e-1,
			Scalar l2_decay = 1e-3, Scalar epsilon = 1e-5) {
		for (std::size_t i = 0; i < 4; ++i)
			check(cattle_hip_layer_param_adam_update(handle, i, (double) learning_rate, (double) l1_decay, (double) l2_decay,
					(double) epsilon, timestep));
	}
	inline void reset_grads() {
		for (std::size_t i = 0; i < 4; ++i)
			check(cattle_hip_layer_reset_param_grad(handle, i));
	}
private:
	cattle_hip_layer_t handle;
	Dims input_dims;
	std::size_t hidden;
	OutputSeqSizeFunc seq;
	bool foremost;
	std::size_t batch, in_len;
};

} /* namespace device */
} /* namespace hip */
} /* namespace cattle */

#endif /* CATTLE_HIP_DEVICENET_HPP_ */
