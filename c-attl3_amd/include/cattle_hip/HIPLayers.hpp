/*
 * HIPLayers.hpp — header-only C++11 layers for C-ATTL3 that run on an MI355X through libcattle_hip.
 *
 * Each class derives from the unchanged cattle::Layer hierarchy (core/Layer.hpp:30-155,
 * layer/KernelLayer.hpp:28-82, layer/ActivationLayer.hpp:26-79), takes the constructor arguments
 * of the CPU layer it stands in for, and keeps ordinary host-side Parameters objects, so any
 * NeuralNetwork, Optimizer or GradientCheck of the library works on top of it unchanged:
 *
 *   cattle::ConvKernelLayer<S,R>        ->  cattle::hip::ConvKernelHIPLayer<S,R>
 *   cattle::TransConvKernelLayer<S,R>   ->  cattle::hip::TransConvKernelHIPLayer<S,R>
 *   cattle::DenseKernelLayer<S,R>       ->  cattle::hip::DenseKernelHIPLayer<S,R>
 *   cattle::BatchNormLayer<S,R,P>       ->  cattle::hip::BatchNormHIPLayer<S,R,P>
 *   cattle::<Name>ActivationLayer<S,R>  ->  cattle::hip::<Name>ActivationHIPLayer<S,R>
 *   cattle::MaxPoolLayer / MeanPoolLayer<S,R> -> cattle::hip::MaxPoolHIPLayer / MeanPoolHIPLayer<S,R>
 *
 * pass_forward / pass_back hand the Eigen tensor's buffer to the C ABI as a HOST buffer; the
 * library stages it through device memory. Parameter values are pushed to the device before every
 * forward pass (the optimizer may have changed them through Parameters::set_values), and the
 * gradient of a backward pass is pulled back and given to Parameters::accumulate_grad, so value
 * and gradient constraints, regularisation and parameter sharing behave exactly as on the CPU.
 *
 * Include after the C-ATTL3 headers are on the include path (the default pulls in "Cattle.hpp");
 * link with -lcattle_hip.
 */
#ifndef CATTLE_HIP_HIPLAYERS_HPP_
#define CATTLE_HIP_HIPLAYERS_HPP_

#ifndef CATTLE_HIP_CATTLE_HEADER
#define CATTLE_HIP_CATTLE_HEADER "Cattle.hpp"
#endif
#include CATTLE_HIP_CATTLE_HEADER

#include <array>
#include <cassert>
#include <cstddef>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "cattle_hip.h"

namespace cattle {
namespace hip {

namespace detail {

inline void check(int status) {
	if (status != CATTLE_HIP_OK)
		throw std::runtime_error(std::string("cattle_hip: ") + cattle_hip_last_error());
}

template<typename Scalar> struct ScalarCode;
template<> struct ScalarCode<float> { static constexpr cattle_hip_dtype value = CATTLE_HIP_F32; };
template<> struct ScalarCode<double> { static constexpr cattle_hip_dtype value = CATTLE_HIP_F64; };

/* Owner of one device-side layer handle. */
class Handle {
public:
	inline Handle() : handle(nullptr) { }
	inline ~Handle() {
		if (handle)
			cattle_hip_layer_destroy(handle);
	}
	Handle(const Handle&) = delete;
	Handle& operator=(const Handle&) = delete;
	inline cattle_hip_layer_t get() const {
		return handle;
	}
	inline cattle_hip_layer_t* out() {
		return &handle;
	}
private:
	cattle_hip_layer_t handle;
};

/* What the device holds of one parameter matrix: the values of the last upload. The host Parameters object stays the
 * owner of the values (optimizers call its set_values), and most passes find it unchanged - every inference pass, the
 * passes of frozen or shared layers, all passes between two optimizer steps - so a pass compares before it uploads: a
 * comparison in host memory costs a fraction of the copy, the wait for it and the re-layout kernel that a new version
 * of the weights triggers. */
template<typename Scalar>
class UploadedValues {
public:
	inline bool differ(const Scalar* values, std::size_t count) const {
		return last.size() != count || std::memcmp(last.data(), values, count * sizeof(Scalar)) != 0;
	}
	inline void remember(const Scalar* values, std::size_t count) {
		last.assign(values, values + count);
	}
private:
	std::vector<Scalar> last;
};

/* Parameters::get_values() -> device, if they are not there already. */
template<typename Scalar>
inline void push_values(cattle_hip_layer_t layer, std::size_t index, const Parameters<Scalar>& params, UploadedValues<Scalar>& uploaded) {
	const Matrix<Scalar>& values = params.get_values();
	assert((std::size_t) values.rows() == params.get_rows() && (std::size_t) values.cols() == params.get_cols());
	const std::size_t count = params.get_rows() * params.get_cols();
	if (!uploaded.differ(values.data(), count))
		return;
	check(cattle_hip_layer_set_param_values(layer, index, values.data(), CATTLE_HIP_HOST));
	uploaded.remember(values.data(), count);
}

/* Device gradient of the last backward pass -> Parameters::accumulate_grad(); the device buffer is
 * cleared so that the host object stays the only accumulator. */
template<typename Scalar>
inline void drain_grad(cattle_hip_layer_t layer, std::size_t index, Parameters<Scalar>& params) {
	if (!params.are_optimizable())
		return;
	Matrix<Scalar> grad(params.get_rows(), params.get_cols());
	check(cattle_hip_layer_get_param_grad(layer, index, grad.data(), CATTLE_HIP_HOST));
	check(cattle_hip_layer_reset_param_grad(layer, index));
	params.accumulate_grad(grad);
}

/* (batch, dims...) as the index array of a rank Rank + 1 tensor. */
template<typename Dims, std::size_t Rank>
inline std::array<std::size_t,Rank + 1> batch_dims(std::size_t batch, const Dims& dims) {
	std::array<std::size_t,Rank + 1> out;
	out[0] = batch;
	for (std::size_t i = 0; i < Rank; ++i)
		out[i + 1] = dims(i);
	return out;
}

template<typename Data, typename Dims, std::size_t Rank>
inline bool dims_match(const Data& data, const Dims& dims) {
	for (std::size_t i = 0; i < Rank; ++i)
		if ((std::size_t) data.dimension(i + 1) != (std::size_t) dims(i))
			return false;
	return true;
}

/* Dimensions::extend<3 - Rank>() spelled out: missing ranks are ones. */
template<typename Dims, std::size_t Rank>
inline std::array<std::size_t,3> extended(const Dims& dims) {
	std::array<std::size_t,3> out = { { 1, 1, 1 } };
	for (std::size_t i = 0; i < Rank; ++i)
		out[i] = dims(i);
	return out;
}

template<typename Dims, std::size_t Rank>
inline Dims contracted(const std::array<std::size_t,3>& ext) {
	std::array<std::size_t,Rank> arr;
	for (std::size_t i = 0; i < Rank; ++i)
		arr[i] = ext[i];
	return Dims(arr);
}

} /* namespace detail */

/**
 * Common body of the drop-ins for ConvKernelLayer<Scalar,Rank> (layer/kernel/ConvKernelLayer.hpp:232-512)
 * and, with Transposed, TransConvKernelLayer<Scalar,Rank> (layer/kernel/TransConvKernelLayer.hpp:241-520).
 * For rank 2 the input is viewed as single-channel, for rank 1 additionally as single-column, and the
 * filters are folded into the last nominal rank of the output, as in calculate_adjusted_output_dims
 * (ConvKernelLayer.hpp:206-217, TransConvKernelLayer.hpp:241-251).
 */
template<typename Scalar, std::size_t Rank, bool Transposed>
class ConvFamilyHIPLayerBase : public KernelLayer<Scalar,Rank> {
	typedef Layer<Scalar,Rank> Root;
	typedef KernelLayer<Scalar,Rank> Base;
public:
	inline Root* clone() const {
		return new ConvFamilyHIPLayerBase(*this, false);
	}
	inline Root* clone_with_shared_params() {
		return new ConvFamilyHIPLayerBase(*this, true);
	}
	inline void empty_cache() {
		detail::check(cattle_hip_layer_empty_cache(device.get()));
	}
	inline typename Root::Data pass_forward(typename Root::Data in, bool training) {
		assert((detail::dims_match<typename Root::Data,typename Root::Dims,Rank>(in, Base::input_dims)));
		assert(in.dimension(0) > 0);
		batch_size = in.dimension(0);
		detail::push_values<Scalar>(device.get(), 0, *Base::weights, uploaded_weights);
		detail::push_values<Scalar>(device.get(), 1, *Base::bias, uploaded_bias);
		typename Root::Data out(detail::batch_dims<typename Root::Dims,Rank>(batch_size, Base::output_dims));
		detail::check(cattle_hip_layer_forward(device.get(), in.data(), CATTLE_HIP_HOST, batch_size, training ? 1 : 0,
				out.data(), CATTLE_HIP_HOST));
		return out;
	}
	inline typename Root::Data pass_back(typename Root::Data out_grad) {
		assert((detail::dims_match<typename Root::Data,typename Root::Dims,Rank>(out_grad, Base::output_dims)));
		assert(out_grad.dimension(0) > 0 && batch_size == (std::size_t) out_grad.dimension(0));
		const bool input_layer = Base::is_input_layer();
		detail::check(cattle_hip_layer_set_input_layer(device.get(), input_layer ? 1 : 0));
		typename Root::Data prev_out_grad;
		if (!input_layer)
			prev_out_grad = typename Root::Data(detail::batch_dims<typename Root::Dims,Rank>(batch_size, Base::input_dims));
		detail::check(cattle_hip_layer_backward(device.get(), out_grad.data(), CATTLE_HIP_HOST, batch_size,
				input_layer ? nullptr : prev_out_grad.data(), CATTLE_HIP_HOST));
		detail::drain_grad<Scalar>(device.get(), 0, *Base::weights);
		detail::drain_grad<Scalar>(device.get(), 1, *Base::bias);
		return prev_out_grad;
	}
protected:
	struct Geometry {
		std::size_t filters, receptor_height, receptor_width, vertical_padding, horizontal_padding, vertical_stride,
				horizontal_stride, vertical_dilation, horizontal_dilation;
	};
	inline ConvFamilyHIPLayerBase(const typename Root::Dims& input_dims, const Geometry& geom,
			ParamsSharedPtr<Scalar> weights, ParamsSharedPtr<Scalar> bias) :
				Base(input_dims, output_dims_for(input_dims, geom), weights, bias),
				geom(geom),
				batch_size(0) {
		create_device_layer();
	}
	inline ConvFamilyHIPLayerBase(const ConvFamilyHIPLayerBase<Scalar,Rank,Transposed>& layer, bool share_params) :
			Base(layer, share_params),
			geom(layer.geom),
			batch_size(0) {
		create_device_layer();
	}
	inline static std::size_t receptor_volume(const typename Root::Dims& input_dims, std::size_t receptor_height,
			std::size_t receptor_width) {
		return receptor_height * receptor_width * detail::extended<typename Root::Dims,Rank>(input_dims)[2];
	}
	inline static std::size_t spatial_output_dim(std::size_t input_dim, std::size_t receptor, std::size_t padding,
			std::size_t dilation, std::size_t stride) {
		if (Transposed)         /* TransConvKernelLayer.hpp:226-229 */
			return (input_dim - 1) * stride + receptor + (receptor - 1) * dilation - 2 * padding;
		return (input_dim - receptor - (receptor - 1) * dilation + 2 * padding) / stride + 1;       /* ConvKernelLayer.hpp:194-197 */
	}
	inline static typename Root::Dims output_dims_for(const typename Root::Dims& input_dims, const Geometry& g) {
		const std::array<std::size_t,3> in = detail::extended<typename Root::Dims,Rank>(input_dims);
		std::array<std::size_t,3> out = { {
				spatial_output_dim(in[0], g.receptor_height, g.vertical_padding, g.vertical_dilation, g.vertical_stride),
				spatial_output_dim(in[1], g.receptor_width, g.horizontal_padding, g.horizontal_dilation, g.horizontal_stride),
				1 } };
		out[Rank - 1] *= g.filters;
		return detail::contracted<typename Root::Dims,Rank>(out);
	}
private:
	inline void create_device_layer() {
		const std::array<std::size_t,3> in = detail::extended<typename Root::Dims,Rank>(Base::input_dims);
		detail::check((Transposed ? cattle_hip_transconv_create : cattle_hip_conv_create)(detail::ScalarCode<Scalar>::value,
				in[0], in[1], in[2], geom.filters, geom.receptor_height, geom.receptor_width, geom.vertical_padding,
				geom.horizontal_padding, geom.vertical_stride, geom.horizontal_stride, geom.vertical_dilation,
				geom.horizontal_dilation, device.out()));
	}
	const Geometry geom;
	detail::Handle device;
	detail::UploadedValues<Scalar> uploaded_weights, uploaded_bias;
	std::size_t batch_size;
};

template<typename Scalar, std::size_t Rank>
using ConvKernelHIPLayerBase = ConvFamilyHIPLayerBase<Scalar,Rank,false>;
template<typename Scalar, std::size_t Rank>
using TransConvKernelHIPLayerBase = ConvFamilyHIPLayerBase<Scalar,Rank,true>;

/** Rank 3 and rank 2: the constructor of ConvKernelLayer<Scalar,3|2> (ConvKernelLayer.hpp:282-296, :375-389). */
template<typename Scalar, std::size_t Rank = 3>
class ConvKernelHIPLayer : public ConvKernelHIPLayerBase<Scalar,Rank> {
	typedef Layer<Scalar,Rank> Root;
	typedef ConvKernelHIPLayerBase<Scalar,Rank> ConvBase;
public:
	inline ConvKernelHIPLayer(const typename Root::Dims& input_dims, std::size_t filters,
			ParamInitSharedPtr<Scalar> weight_init, std::size_t receptor_height = 3, std::size_t receptor_width = 3,
			std::size_t vertical_padding = 1, std::size_t horizontal_padding = 1, std::size_t vertical_stride = 1,
			std::size_t horizontal_stride = 1, std::size_t vertical_dilation = 0, std::size_t horizontal_dilation = 0,
			ParamRegSharedPtr<Scalar> weight_reg = nullptr, Scalar weight_clip = 0, Scalar weight_max_l1_norm = 0,
			Scalar weight_max_l2_norm = 0, Scalar weight_grad_clip = 0, Scalar weight_grad_max_l1_norm = 0,
			Scalar weight_grad_max_l2_norm = 0, ParamRegSharedPtr<Scalar> bias_reg = nullptr, Scalar bias_clip = 0,
			Scalar bias_max_l1_norm = 0, Scalar bias_max_l2_norm = 0, Scalar bias_grad_clip = 0,
			Scalar bias_grad_max_l1_norm = 0, Scalar bias_grad_max_l2_norm = 0) :
				ConvBase(input_dims, typename ConvBase::Geometry{ filters, receptor_height, receptor_width, vertical_padding,
						horizontal_padding, vertical_stride, horizontal_stride, vertical_dilation, horizontal_dilation },
						std::make_shared<StandardParameters<Scalar>>(ConvBase::receptor_volume(input_dims, receptor_height,
								receptor_width), filters, true, weight_init, weight_reg, weight_clip, weight_max_l1_norm,
								weight_max_l2_norm, weight_grad_clip, weight_grad_max_l1_norm, weight_grad_max_l2_norm),
						std::make_shared<StandardParameters<Scalar>>(1, filters, true,
								std::make_shared<ZeroParameterInitialization<Scalar>>(), bias_reg, bias_clip, bias_max_l1_norm,
								bias_max_l2_norm, bias_grad_clip, bias_grad_max_l1_norm, bias_grad_max_l2_norm)) {
		static_assert(Rank == 2 || Rank == 3, "rank 1 has its own constructor");
	}
};

/** Rank 1: the constructor of ConvKernelLayer<Scalar,1> (ConvKernelLayer.hpp:462-478). */
template<typename Scalar>
class ConvKernelHIPLayer<Scalar,1> : public ConvKernelHIPLayerBase<Scalar,1> {
	typedef Layer<Scalar,1> Root;
	typedef ConvKernelHIPLayerBase<Scalar,1> ConvBase;
public:
	inline ConvKernelHIPLayer(const typename Root::Dims& input_dims, std::size_t filters,
			ParamInitSharedPtr<Scalar> weight_init, std::size_t receptor_length = 3, std::size_t padding = 1,
			std::size_t stride = 1, std::size_t dilation = 0, ParamRegSharedPtr<Scalar> weight_reg = nullptr,
			Scalar weight_clip = 0, Scalar weight_max_l1_norm = 0, Scalar weight_max_l2_norm = 0,
			Scalar weight_grad_clip = 0, Scalar weight_grad_max_l1_norm = 0, Scalar weight_grad_max_l2_norm = 0,
			ParamRegSharedPtr<Scalar> bias_reg = nullptr, Scalar bias_clip = 0, Scalar bias_max_l1_norm = 0,
			Scalar bias_max_l2_norm = 0, Scalar bias_grad_clip = 0, Scalar bias_grad_max_l1_norm = 0,
			Scalar bias_grad_max_l2_norm = 0) :
				ConvBase(input_dims, typename ConvBase::Geometry{ filters, receptor_length, 1, padding, 0, stride, 1, dilation, 0 },
						std::make_shared<StandardParameters<Scalar>>(ConvBase::receptor_volume(input_dims, receptor_length, 1),
								filters, true, weight_init, weight_reg, weight_clip, weight_max_l1_norm, weight_max_l2_norm,
								weight_grad_clip, weight_grad_max_l1_norm, weight_grad_max_l2_norm),
						std::make_shared<StandardParameters<Scalar>>(1, filters, true,
								std::make_shared<ZeroParameterInitialization<Scalar>>(), bias_reg, bias_clip, bias_max_l1_norm,
								bias_max_l2_norm, bias_grad_clip, bias_grad_max_l1_norm, bias_grad_max_l2_norm)) { }
};

/**
 * Drop-in for TransConvKernelLayer<Scalar,3|2> (TransConvKernelLayer.hpp:290-304, :386-400): weights
 * [channels x receptor_height*receptor_width*filters], one bias entry per output activation (:46-56).
 */
template<typename Scalar, std::size_t Rank = 3>
class TransConvKernelHIPLayer : public TransConvKernelHIPLayerBase<Scalar,Rank> {
	typedef Layer<Scalar,Rank> Root;
	typedef TransConvKernelHIPLayerBase<Scalar,Rank> TransBase;
public:
	inline TransConvKernelHIPLayer(const typename Root::Dims& input_dims, std::size_t filters,
			ParamInitSharedPtr<Scalar> weight_init, std::size_t receptor_height = 3, std::size_t receptor_width = 3,
			std::size_t vertical_padding = 1, std::size_t horizontal_padding = 1, std::size_t vertical_stride = 1,
			std::size_t horizontal_stride = 1, std::size_t vertical_dilation = 0, std::size_t horizontal_dilation = 0,
			ParamRegSharedPtr<Scalar> weight_reg = nullptr, Scalar weight_clip = 0, Scalar weight_max_l1_norm = 0,
			Scalar weight_max_l2_norm = 0, Scalar weight_grad_clip = 0, Scalar weight_grad_max_l1_norm = 0,
			Scalar weight_grad_max_l2_norm = 0, ParamRegSharedPtr<Scalar> bias_reg = nullptr, Scalar bias_clip = 0,
			Scalar bias_max_l1_norm = 0, Scalar bias_max_l2_norm = 0, Scalar bias_grad_clip = 0,
			Scalar bias_grad_max_l1_norm = 0, Scalar bias_grad_max_l2_norm = 0) :
				TransBase(input_dims, typename TransBase::Geometry{ filters, receptor_height, receptor_width, vertical_padding,
						horizontal_padding, vertical_stride, horizontal_stride, vertical_dilation, horizontal_dilation },
						std::make_shared<StandardParameters<Scalar>>(detail::extended<typename Root::Dims,Rank>(input_dims)[2],
								receptor_height * receptor_width * filters, true, weight_init, weight_reg, weight_clip,
								weight_max_l1_norm, weight_max_l2_norm, weight_grad_clip, weight_grad_max_l1_norm,
								weight_grad_max_l2_norm),
						std::make_shared<StandardParameters<Scalar>>(1, TransBase::output_dims_for(input_dims,
								typename TransBase::Geometry{ filters, receptor_height, receptor_width, vertical_padding,
										horizontal_padding, vertical_stride, horizontal_stride, vertical_dilation,
										horizontal_dilation }).get_volume(), true,
								std::make_shared<ZeroParameterInitialization<Scalar>>(), bias_reg, bias_clip, bias_max_l1_norm,
								bias_max_l2_norm, bias_grad_clip, bias_grad_max_l1_norm, bias_grad_max_l2_norm)) {
		static_assert(Rank == 2 || Rank == 3, "rank 1 has its own constructor");
	}
};

/** Rank 1: the constructor of TransConvKernelLayer<Scalar,1> (TransConvKernelLayer.hpp:482-495). */
template<typename Scalar>
class TransConvKernelHIPLayer<Scalar,1> : public TransConvKernelHIPLayerBase<Scalar,1> {
	typedef Layer<Scalar,1> Root;
	typedef TransConvKernelHIPLayerBase<Scalar,1> TransBase;
public:
	inline TransConvKernelHIPLayer(const typename Root::Dims& input_dims, std::size_t filters,
			ParamInitSharedPtr<Scalar> weight_init, std::size_t receptor_length = 3, std::size_t padding = 1,
			std::size_t stride = 1, std::size_t dilation = 0, ParamRegSharedPtr<Scalar> weight_reg = nullptr,
			Scalar weight_clip = 0, Scalar weight_max_l1_norm = 0, Scalar weight_max_l2_norm = 0,
			Scalar weight_grad_clip = 0, Scalar weight_grad_max_l1_norm = 0, Scalar weight_grad_max_l2_norm = 0,
			ParamRegSharedPtr<Scalar> bias_reg = nullptr, Scalar bias_clip = 0, Scalar bias_max_l1_norm = 0,
			Scalar bias_max_l2_norm = 0, Scalar bias_grad_clip = 0, Scalar bias_grad_max_l1_norm = 0,
			Scalar bias_grad_max_l2_norm = 0) :
				TransBase(input_dims, typename TransBase::Geometry{ filters, receptor_length, 1, padding, 0, stride, 1, dilation, 0 },
						std::make_shared<StandardParameters<Scalar>>(1, receptor_length * filters, true, weight_init, weight_reg,
								weight_clip, weight_max_l1_norm, weight_max_l2_norm, weight_grad_clip, weight_grad_max_l1_norm,
								weight_grad_max_l2_norm),
						std::make_shared<StandardParameters<Scalar>>(1, TransBase::output_dims_for(input_dims,
								typename TransBase::Geometry{ filters, receptor_length, 1, padding, 0, stride, 1, dilation, 0 })
								.get_volume(), true, std::make_shared<ZeroParameterInitialization<Scalar>>(), bias_reg, bias_clip,
								bias_max_l1_norm, bias_max_l2_norm, bias_grad_clip, bias_grad_max_l1_norm, bias_grad_max_l2_norm)) { }
};

/** Drop-in for DenseKernelLayer<Scalar,Rank> (layer/kernel/DenseKernelLayer.hpp:27-120). */
template<typename Scalar, std::size_t Rank = 1>
class DenseKernelHIPLayer : public KernelLayer<Scalar,Rank> {
	typedef Layer<Scalar,Rank> Root;
	typedef KernelLayer<Scalar,Rank> Base;
public:
	inline DenseKernelHIPLayer(const typename Root::Dims& input_dims, std::size_t output_size,
			ParamInitSharedPtr<Scalar> weight_init, ParamRegSharedPtr<Scalar> weight_reg = nullptr,
			Scalar weight_clip = 0, Scalar weight_max_l1_norm = 0, Scalar weight_max_l2_norm = 0,
			Scalar weight_grad_clip = 0, Scalar weight_grad_max_l1_norm = 0, Scalar weight_grad_max_l2_norm = 0,
			ParamRegSharedPtr<Scalar> bias_reg = nullptr, Scalar bias_clip = 0, Scalar bias_max_l1_norm = 0,
			Scalar bias_max_l2_norm = 0, Scalar bias_grad_clip = 0, Scalar bias_grad_max_l1_norm = 0,
			Scalar bias_grad_max_l2_norm = 0) :
				Base(input_dims, output_dims_for(output_size),
						std::make_shared<StandardParameters<Scalar>>(input_dims.get_volume(), output_size, true,
								weight_init, weight_reg, weight_clip, weight_max_l1_norm, weight_max_l2_norm,
								weight_grad_clip, weight_grad_max_l1_norm, weight_grad_max_l2_norm),
						std::make_shared<StandardParameters<Scalar>>(1, output_size, true,
								std::make_shared<ZeroParameterInitialization<Scalar>>(), bias_reg, bias_clip,
								bias_max_l1_norm, bias_max_l2_norm, bias_grad_clip, bias_grad_max_l1_norm,
								bias_grad_max_l2_norm)),
				batch_size(0) {
		create_device_layer();
	}
	inline DenseKernelHIPLayer(const DenseKernelHIPLayer<Scalar,Rank>& layer, bool share_params = false) :
			Base(layer, share_params),
			batch_size(0) {
		create_device_layer();
	}
	inline Root* clone() const {
		return new DenseKernelHIPLayer(*this);
	}
	inline Root* clone_with_shared_params() {
		return new DenseKernelHIPLayer(*this, true);
	}
	inline void empty_cache() {
		detail::check(cattle_hip_layer_empty_cache(device.get()));
	}
	inline typename Root::Data pass_forward(typename Root::Data in, bool training) {
		assert((detail::dims_match<typename Root::Data,typename Root::Dims,Rank>(in, Base::input_dims)));
		assert(in.dimension(0) > 0);
		batch_size = in.dimension(0);
		detail::push_values<Scalar>(device.get(), 0, *Base::weights, uploaded_weights);
		detail::push_values<Scalar>(device.get(), 1, *Base::bias, uploaded_bias);
		typename Root::Data out(detail::batch_dims<typename Root::Dims,Rank>(batch_size, Base::output_dims));
		detail::check(cattle_hip_layer_forward(device.get(), in.data(), CATTLE_HIP_HOST, batch_size, training ? 1 : 0,
				out.data(), CATTLE_HIP_HOST));
		return out;
	}
	inline typename Root::Data pass_back(typename Root::Data out_grad) {
		assert((detail::dims_match<typename Root::Data,typename Root::Dims,Rank>(out_grad, Base::output_dims)));
		assert(out_grad.dimension(0) > 0 && batch_size == (std::size_t) out_grad.dimension(0));
		const bool input_layer = Base::is_input_layer();
		detail::check(cattle_hip_layer_set_input_layer(device.get(), input_layer ? 1 : 0));
		typename Root::Data prev_out_grad;
		if (!input_layer)
			prev_out_grad = typename Root::Data(detail::batch_dims<typename Root::Dims,Rank>(batch_size, Base::input_dims));
		detail::check(cattle_hip_layer_backward(device.get(), out_grad.data(), CATTLE_HIP_HOST, batch_size,
				input_layer ? nullptr : prev_out_grad.data(), CATTLE_HIP_HOST));
		detail::drain_grad<Scalar>(device.get(), 0, *Base::weights);
		detail::drain_grad<Scalar>(device.get(), 1, *Base::bias);
		return prev_out_grad;
	}
private:
	inline static typename Root::Dims output_dims_for(std::size_t output_size) {
		std::array<std::size_t,3> ext = { { output_size, 1, 1 } };      /* Base(input_dims, { output_size }, ...) */
		return detail::contracted<typename Root::Dims,Rank>(ext);
	}
	inline void create_device_layer() {
		detail::check(cattle_hip_dense_create(detail::ScalarCode<Scalar>::value, Base::input_dims.get_volume(),
				Base::output_dims.get_volume(), device.out()));
	}
	detail::Handle device;
	detail::UploadedValues<Scalar> uploaded_weights, uploaded_bias;
	std::size_t batch_size;
};

/**
 * Drop-in for BatchNormLayer<Scalar,Rank,PerLastRank> (layer/BatchNormLayer.hpp:27-293 per last
 * rank, :296-470 per activation). get_params() has the reference's order and shapes: per last
 * rank, four 1x1 matrices per channel (running mean, running inverse sd, gamma, beta, :263-272);
 * per activation, four 1 x volume row vectors (:399-406).
 */
template<typename Scalar, std::size_t Rank, bool PerLastRank = (Rank == 3)>
class BatchNormHIPLayer : public Layer<Scalar,Rank> {
	typedef Layer<Scalar,Rank> Base;
	typedef BatchNormHIPLayer<Scalar,Rank,PerLastRank> Self;
	typedef std::shared_ptr<StandardParameters<Scalar>> StdParamsSharedPtr;
public:
	inline BatchNormHIPLayer(const typename Base::Dims& dims, Scalar norm_avg_decay = .1,
			Scalar epsilon = NumericUtils<Scalar>::EPSILON2, ParamRegSharedPtr<Scalar> gamma_reg = nullptr,
			Scalar gamma_clip = 0, Scalar gamma_max_l1_norm = 0, Scalar gamma_max_l2_norm = 0,
			Scalar gamma_grad_clip = 0, Scalar gamma_grad_max_l1_norm = 0, Scalar gamma_grad_max_l2_norm = 0,
			ParamRegSharedPtr<Scalar> beta_reg = nullptr, Scalar beta_clip = 0, Scalar beta_max_l1_norm = 0,
			Scalar beta_max_l2_norm = 0, Scalar beta_grad_clip = 0, Scalar beta_grad_max_l1_norm = 0,
			Scalar beta_grad_max_l2_norm = 0) :
				owner(*this),
				dims(dims),
				norm_avg_decay(norm_avg_decay),
				epsilon(epsilon),
				groups(PerLastRank ? dims(Rank - 1) : dims.get_volume()),
				param_cols(PerLastRank ? 1 : dims.get_volume()),
				input_layer(false),
				avgs_init(false),
				batch_size(0) {
		auto gamma_init = std::make_shared<OneParameterInitialization<Scalar>>();
		auto beta_init = std::make_shared<ZeroParameterInitialization<Scalar>>();
		const std::size_t sets = PerLastRank ? groups : 1;
		for (std::size_t i = 0; i < sets; ++i) {
			avg_means.push_back(std::make_shared<StandardParameters<Scalar>>(1, param_cols, false));
			avg_inv_sds.push_back(std::make_shared<StandardParameters<Scalar>>(1, param_cols, false));
			gammas.push_back(std::make_shared<StandardParameters<Scalar>>(1, param_cols, true, gamma_init, gamma_reg,
					gamma_clip, gamma_max_l1_norm, gamma_max_l2_norm, gamma_grad_clip, gamma_grad_max_l1_norm,
					gamma_grad_max_l2_norm));
			betas.push_back(std::make_shared<StandardParameters<Scalar>>(1, param_cols, true, beta_init, beta_reg,
					beta_clip, beta_max_l1_norm, beta_max_l2_norm, beta_grad_clip, beta_grad_max_l1_norm,
					beta_grad_max_l2_norm));
		}
		create_device_layer();
	}
	inline BatchNormHIPLayer(const Self& layer, bool share_params = false) :
			owner(share_params ? layer.owner : *this),
			dims(layer.dims),
			norm_avg_decay(layer.norm_avg_decay),
			epsilon(layer.epsilon),
			groups(layer.groups),
			param_cols(layer.param_cols),
			input_layer(layer.input_layer),
			avgs_init(layer.avgs_init),
			batch_size(0) {
		copy_params(layer.avg_means, avg_means, share_params);
		copy_params(layer.avg_inv_sds, avg_inv_sds, share_params);
		copy_params(layer.gammas, gammas, share_params);
		copy_params(layer.betas, betas, share_params);
		create_device_layer();
	}
	inline Base* clone() const {
		return new BatchNormHIPLayer(*this);
	}
	inline Base* clone_with_shared_params() {
		return new BatchNormHIPLayer(*this, true);
	}
	inline const Base& get_params_owner() const {
		return owner;
	}
	inline const typename Base::Dims& get_input_dims() const {
		return dims;
	}
	inline const typename Base::Dims& get_output_dims() const {
		return dims;
	}
	inline bool is_input_layer() const {
		return input_layer;
	}
	inline void set_input_layer(bool input_layer) {
		this->input_layer = input_layer;
	}
	inline std::vector<const Parameters<Scalar>*> get_params() const {
		std::vector<const Parameters<Scalar>*> params_vec;
		for (std::size_t i = 0; i < avg_means.size(); ++i) {
			params_vec.push_back(avg_means[i].get());
			params_vec.push_back(avg_inv_sds[i].get());
			params_vec.push_back(gammas[i].get());
			params_vec.push_back(betas[i].get());
		}
		return params_vec;
	}
	inline std::vector<Parameters<Scalar>*> get_params() {
		std::vector<Parameters<Scalar>*> params_vec;
		for (std::size_t i = 0; i < avg_means.size(); ++i) {
			params_vec.push_back(avg_means[i].get());
			params_vec.push_back(avg_inv_sds[i].get());
			params_vec.push_back(gammas[i].get());
			params_vec.push_back(betas[i].get());
		}
		return params_vec;
	}
	inline void empty_cache() {
		detail::check(cattle_hip_layer_empty_cache(device.get()));
	}
	inline typename Base::Data pass_forward(typename Base::Data in, bool training) {
		assert((detail::dims_match<typename Base::Data,typename Base::Dims,Rank>(in, dims)));
		assert(in.dimension(0) > 0);
		assert(training || avgs_init);
		batch_size = in.dimension(0);
		push(2, gammas);
		push(3, betas);
		if (avgs_init) {
			push(0, avg_means);
			push(1, avg_inv_sds);
		}
		detail::check(cattle_hip_batchnorm_set_stats_initialized(device.get(), avgs_init ? 1 : 0));
		typename Base::Data out(detail::batch_dims<typename Base::Dims,Rank>(batch_size, dims));
		detail::check(cattle_hip_layer_forward(device.get(), in.data(), CATTLE_HIP_HOST, batch_size, training ? 1 : 0,
				out.data(), CATTLE_HIP_HOST));
		if (training) {
			/* the running statistics are maintained through set_values, as in the reference (:234-243) */
			pull_values(0, avg_means);
			pull_values(1, avg_inv_sds);
			avgs_init = true;
		}
		return out;
	}
	inline typename Base::Data pass_back(typename Base::Data out_grad) {
		assert((detail::dims_match<typename Base::Data,typename Base::Dims,Rank>(out_grad, dims)));
		assert(out_grad.dimension(0) > 0 && batch_size == (std::size_t) out_grad.dimension(0));
		detail::check(cattle_hip_layer_set_input_layer(device.get(), input_layer ? 1 : 0));
		typename Base::Data prev_out_grad;
		if (!input_layer)
			prev_out_grad = typename Base::Data(detail::batch_dims<typename Base::Dims,Rank>(batch_size, dims));
		detail::check(cattle_hip_layer_backward(device.get(), out_grad.data(), CATTLE_HIP_HOST, batch_size,
				input_layer ? nullptr : prev_out_grad.data(), CATTLE_HIP_HOST));
		pull_grads(2, gammas);
		pull_grads(3, betas);
		return prev_out_grad;
	}
private:
	typedef std::vector<StdParamsSharedPtr> ParamSet;
	inline static void copy_params(const ParamSet& from, ParamSet& to, bool share) {
		for (std::size_t i = 0; i < from.size(); ++i)
			to.push_back(share ? from[i] : StdParamsSharedPtr(static_cast<StandardParameters<Scalar>*>(from[i]->clone())));
	}
	inline void create_device_layer() {
		/* the statistics group is the last nominal rank: hand it over as the channel rank */
		std::size_t h = 1, w = 1, c = 1;
		if (PerLastRank) {
			h = dims.get_volume() / groups;
			c = groups;
		} else {
			h = dims.get_volume();
		}
		detail::check(cattle_hip_batchnorm_create(detail::ScalarCode<Scalar>::value, h, w, c, PerLastRank ? 1 : 0,
				(double) norm_avg_decay, (double) epsilon, device.out()));
	}
	/* host Parameters (one 1x1 per channel, or one row vector) <-> the device's 1 x groups row */
	inline void push(std::size_t index, const ParamSet& set) {
		Matrix<Scalar> row(1, groups);
		for (std::size_t i = 0; i < set.size(); ++i)
			for (std::size_t j = 0; j < param_cols; ++j)
				row(0, i * param_cols + j) = set[i]->get_values()(0, j);
		if (!uploaded[index].differ(row.data(), groups))
			return;
		detail::check(cattle_hip_layer_set_param_values(device.get(), index, row.data(), CATTLE_HIP_HOST));
		uploaded[index].remember(row.data(), groups);
	}
	inline void pull_values(std::size_t index, ParamSet& set) {
		Matrix<Scalar> row(1, groups);
		detail::check(cattle_hip_layer_get_param_values(device.get(), index, row.data(), CATTLE_HIP_HOST));
		uploaded[index].remember(row.data(), groups);          /* host and device agree from here on */
		for (std::size_t i = 0; i < set.size(); ++i) {
			Matrix<Scalar> part(1, param_cols);
			for (std::size_t j = 0; j < param_cols; ++j)
				part(0, j) = row(0, i * param_cols + j);
			set[i]->set_values(part);
		}
	}
	inline void pull_grads(std::size_t index, ParamSet& set) {
		Matrix<Scalar> row(1, groups);
		detail::check(cattle_hip_layer_get_param_grad(device.get(), index, row.data(), CATTLE_HIP_HOST));
		detail::check(cattle_hip_layer_reset_param_grad(device.get(), index));
		for (std::size_t i = 0; i < set.size(); ++i) {
			Matrix<Scalar> part(1, param_cols);
			for (std::size_t j = 0; j < param_cols; ++j)
				part(0, j) = row(0, i * param_cols + j);
			set[i]->accumulate_grad(part);
		}
	}
	const Self& owner;
	const typename Base::Dims dims;
	const Scalar norm_avg_decay, epsilon;
	const std::size_t groups, param_cols;
	bool input_layer, avgs_init;
	std::size_t batch_size;
	ParamSet avg_means, avg_inv_sds, gammas, betas;
	detail::UploadedValues<Scalar> uploaded[4];
	detail::Handle device;
};

/**
 * Common body of the activation drop-ins (layer/ActivationLayer.hpp:26-79 and
 * layer/activation/<Name>ActivationLayer.hpp). Kind selects the function; param is its scalar
 * hyper-parameter; parametric kinds (PReLU, PSwish) own a 1 x volume StandardParameters.
 */
template<typename Scalar, std::size_t Rank, cattle_hip_activation Kind>
class ActivationHIPLayer : public ActivationLayer<Scalar,Rank> {
	typedef Layer<Scalar,Rank> Root;
	typedef ActivationLayer<Scalar,Rank> Base;
	typedef ActivationHIPLayer<Scalar,Rank,Kind> Self;
public:
	inline ActivationHIPLayer(const typename Root::Dims& dims, Scalar param = 0, ParamsSharedPtr<Scalar> params = nullptr) :
			Base(dims, params),
			param(param),
			batch_size(0) {
		create_device_layer();
	}
	inline ActivationHIPLayer(const Self& layer, bool share_params = false) :
			Base(layer, share_params),
			param(layer.param),
			batch_size(0) {
		create_device_layer();
	}
	inline Root* clone() const {
		return new Self(*this);
	}
	inline Root* clone_with_shared_params() {
		return new Self(*this, true);
	}
	inline void empty_cache() {
		detail::check(cattle_hip_layer_empty_cache(device.get()));
	}
	inline typename Root::Data pass_forward(typename Root::Data in, bool training) {
		assert((detail::dims_match<typename Root::Data,typename Root::Dims,Rank>(in, Base::dims)));
		assert(in.dimension(0) > 0);
		batch_size = in.dimension(0);
		if (Base::params)
			detail::push_values<Scalar>(device.get(), 0, *Base::params, uploaded_params);
		typename Root::Data out(detail::batch_dims<typename Root::Dims,Rank>(batch_size, Base::dims));
		detail::check(cattle_hip_layer_forward(device.get(), in.data(), CATTLE_HIP_HOST, batch_size, training ? 1 : 0,
				out.data(), CATTLE_HIP_HOST));
		return out;
	}
	inline typename Root::Data pass_back(typename Root::Data out_grad) {
		assert((detail::dims_match<typename Root::Data,typename Root::Dims,Rank>(out_grad, Base::dims)));
		assert(out_grad.dimension(0) > 0 && batch_size == (std::size_t) out_grad.dimension(0));
		/* PReLU ignores the input-layer flag (PReLUActivationLayer.hpp:87-109) */
		const bool skip = Base::is_input_layer() && Kind != CATTLE_HIP_ACT_PRELU;
		detail::check(cattle_hip_layer_set_input_layer(device.get(), Base::is_input_layer() ? 1 : 0));
		typename Root::Data prev_out_grad;
		if (!skip)
			prev_out_grad = typename Root::Data(detail::batch_dims<typename Root::Dims,Rank>(batch_size, Base::dims));
		detail::check(cattle_hip_layer_backward(device.get(), out_grad.data(), CATTLE_HIP_HOST, batch_size,
				skip ? nullptr : prev_out_grad.data(), CATTLE_HIP_HOST));
		if (Base::params)
			detail::drain_grad<Scalar>(device.get(), 0, *Base::params);
		return prev_out_grad;
	}
private:
	inline void create_device_layer() {
		detail::check(cattle_hip_activation_create(detail::ScalarCode<Scalar>::value, Kind, Base::dims.get_volume(),
				(double) param, device.out()));
	}
	const Scalar param;
	detail::UploadedValues<Scalar> uploaded_params;
	detail::Handle device;
	std::size_t batch_size;
};

#define CATTLE_HIP_SIMPLE_ACTIVATION(Name, Kind) \
template<typename Scalar, std::size_t Rank> \
class Name##ActivationHIPLayer : public ActivationHIPLayer<Scalar,Rank,Kind> { \
public: \
	inline Name##ActivationHIPLayer(const typename Layer<Scalar,Rank>::Dims& dims) : \
			ActivationHIPLayer<Scalar,Rank,Kind>(dims) { } \
};

#define CATTLE_HIP_SCALAR_ACTIVATION(Name, Kind, arg, def) \
template<typename Scalar, std::size_t Rank> \
class Name##ActivationHIPLayer : public ActivationHIPLayer<Scalar,Rank,Kind> { \
public: \
	inline Name##ActivationHIPLayer(const typename Layer<Scalar,Rank>::Dims& dims, Scalar arg = def) : \
			ActivationHIPLayer<Scalar,Rank,Kind>(dims, arg) { } \
};

CATTLE_HIP_SIMPLE_ACTIVATION(Identity, CATTLE_HIP_ACT_IDENTITY)          /* IdentityActivationLayer.hpp:28-32 */
CATTLE_HIP_SIMPLE_ACTIVATION(BinaryStep, CATTLE_HIP_ACT_BINARY_STEP)     /* BinaryStepActivationLayer.hpp:33-37 */
CATTLE_HIP_SIMPLE_ACTIVATION(Sigmoid, CATTLE_HIP_ACT_SIGMOID)            /* SigmoidActivationLayer.hpp:29-33 */
CATTLE_HIP_SIMPLE_ACTIVATION(Tanh, CATTLE_HIP_ACT_TANH)                  /* TanhActivationLayer.hpp:29-33 */
CATTLE_HIP_SIMPLE_ACTIVATION(Softsign, CATTLE_HIP_ACT_SOFTSIGN)          /* SoftsignActivationLayer.hpp:30-34 */
CATTLE_HIP_SIMPLE_ACTIVATION(Softplus, CATTLE_HIP_ACT_SOFTPLUS)          /* SoftplusActivationLayer.hpp:31-35 */
CATTLE_HIP_SIMPLE_ACTIVATION(ReLU, CATTLE_HIP_ACT_RELU)                  /* ReLUActivationLayer.hpp:36-40 */
CATTLE_HIP_SCALAR_ACTIVATION(Scaled, CATTLE_HIP_ACT_SCALED, scale, 1)    /* ScaledActivationLayer.hpp:28-33 */
CATTLE_HIP_SCALAR_ACTIVATION(LeakyReLU, CATTLE_HIP_ACT_LEAKY_RELU, alpha, 1e-1)   /* LeakyReLUActivationLayer.hpp:40-45 */
CATTLE_HIP_SCALAR_ACTIVATION(ELU, CATTLE_HIP_ACT_ELU, alpha, 1)          /* ELUActivationLayer.hpp:41-47 */
CATTLE_HIP_SCALAR_ACTIVATION(Swish, CATTLE_HIP_ACT_SWISH, beta, 1)       /* SwishActivationLayer.hpp:33-38 */
CATTLE_HIP_SCALAR_ACTIVATION(Softmax, CATTLE_HIP_ACT_SOFTMAX, epsilon, NumericUtils<Scalar>::EPSILON2)   /* SoftmaxActivationLayer.hpp:38-43 */

#undef CATTLE_HIP_SIMPLE_ACTIVATION
#undef CATTLE_HIP_SCALAR_ACTIVATION

/** Drop-in for PReLUActivationLayer<Scalar,Rank> (layer/activation/PReLUActivationLayer.hpp:58-71). */
template<typename Scalar, std::size_t Rank>
class PReLUActivationHIPLayer : public ActivationHIPLayer<Scalar,Rank,CATTLE_HIP_ACT_PRELU> {
public:
	inline PReLUActivationHIPLayer(const typename Layer<Scalar,Rank>::Dims& dims, Scalar init_alpha = 1e-1,
			ParamRegSharedPtr<Scalar> alpha_reg = nullptr, Scalar alpha_clip = 0, Scalar alpha_max_l1_norm = 0,
			Scalar alpha_max_l2_norm = 0, Scalar alpha_grad_clip = 0, Scalar alpha_grad_max_l1_norm = 0,
			Scalar alpha_grad_max_l2_norm = 0) :
				ActivationHIPLayer<Scalar,Rank,CATTLE_HIP_ACT_PRELU>(dims, init_alpha,
						std::make_shared<StandardParameters<Scalar>>(1, dims.get_volume(), true,
								std::make_shared<ConstantParameterInitialization<Scalar>>(init_alpha), alpha_reg, alpha_clip,
								alpha_max_l1_norm, alpha_max_l2_norm, alpha_grad_clip, alpha_grad_max_l1_norm,
								alpha_grad_max_l2_norm)) { }
};

/** Drop-in for PSwishActivationLayer<Scalar,Rank> (layer/activation/PSwishActivationLayer.hpp:55-69). */
template<typename Scalar, std::size_t Rank>
class PSwishActivationHIPLayer : public ActivationHIPLayer<Scalar,Rank,CATTLE_HIP_ACT_PSWISH> {
public:
	inline PSwishActivationHIPLayer(const typename Layer<Scalar,Rank>::Dims& dims, Scalar init_beta = 1,
			ParamRegSharedPtr<Scalar> beta_reg = nullptr, Scalar beta_clip = 0, Scalar beta_max_l1_norm = 0,
			Scalar beta_max_l2_norm = 0, Scalar beta_grad_clip = 0, Scalar beta_grad_max_l1_norm = 0,
			Scalar beta_grad_max_l2_norm = 0) :
				ActivationHIPLayer<Scalar,Rank,CATTLE_HIP_ACT_PSWISH>(dims, init_beta,
						std::make_shared<StandardParameters<Scalar>>(1, dims.get_volume(), true,
								std::make_shared<ConstantParameterInitialization<Scalar>>(init_beta), beta_reg, beta_clip,
								beta_max_l1_norm, beta_max_l2_norm, beta_grad_clip, beta_grad_max_l1_norm,
								beta_grad_max_l2_norm)) { }
};

/**
 * Drop-in for MaxPoolLayer / MeanPoolLayer<Scalar,Rank> (layer/pool/MaxPoolLayer.hpp:89-218,
 * layer/pool/MeanPoolLayer.hpp:47-175, base layer/PoolLayer.hpp:22-157). Rank 2 is viewed as one
 * channel; rank 1 takes (dims, receptor_length, stride) through the specialisations below.
 */
template<typename Scalar, std::size_t Rank, cattle_hip_pool Kind>
class PoolHIPLayer : public Layer<Scalar,Rank> {
	typedef Layer<Scalar,Rank> Base;
	typedef PoolHIPLayer<Scalar,Rank,Kind> Self;
public:
	inline PoolHIPLayer(const typename Base::Dims& input_dims, std::size_t receptor_height, std::size_t receptor_width,
			std::size_t vertical_stride, std::size_t horizontal_stride) :
				input_dims(input_dims),
				output_dims(output_dims_for(input_dims, receptor_height, receptor_width, vertical_stride, horizontal_stride)),
				receptor_height(receptor_height),
				receptor_width(receptor_width),
				vertical_stride(vertical_stride),
				horizontal_stride(horizontal_stride),
				input_layer(false),
				batch_size(0) {
		create_device_layer();
	}
	inline PoolHIPLayer(const Self& layer) :
			input_dims(layer.input_dims),
			output_dims(layer.output_dims),
			receptor_height(layer.receptor_height),
			receptor_width(layer.receptor_width),
			vertical_stride(layer.vertical_stride),
			horizontal_stride(layer.horizontal_stride),
			input_layer(layer.input_layer),
			batch_size(0) {
		create_device_layer();
	}
	inline Base* clone() const {
		return new Self(*this);
	}
	inline Base* clone_with_shared_params() {
		return clone();
	}
	inline const Base& get_params_owner() const {
		return *this;
	}
	inline const typename Base::Dims& get_input_dims() const {
		return input_dims;
	}
	inline const typename Base::Dims& get_output_dims() const {
		return output_dims;
	}
	inline bool is_input_layer() const {
		return input_layer;
	}
	inline void set_input_layer(bool input_layer) {
		this->input_layer = input_layer;
	}
	inline std::vector<const Parameters<Scalar>*> get_params() const {
		return std::vector<const Parameters<Scalar>*>(0);
	}
	inline std::vector<Parameters<Scalar>*> get_params() {
		return std::vector<Parameters<Scalar>*>(0);
	}
	inline void empty_cache() {
		detail::check(cattle_hip_layer_empty_cache(device.get()));
	}
	inline typename Base::Data pass_forward(typename Base::Data in, bool training) {
		assert((detail::dims_match<typename Base::Data,typename Base::Dims,Rank>(in, input_dims)));
		assert(in.dimension(0) > 0);
		batch_size = in.dimension(0);
		typename Base::Data out(detail::batch_dims<typename Base::Dims,Rank>(batch_size, output_dims));
		detail::check(cattle_hip_layer_forward(device.get(), in.data(), CATTLE_HIP_HOST, batch_size, training ? 1 : 0,
				out.data(), CATTLE_HIP_HOST));
		return out;
	}
	inline typename Base::Data pass_back(typename Base::Data out_grad) {
		assert((detail::dims_match<typename Base::Data,typename Base::Dims,Rank>(out_grad, output_dims)));
		assert(out_grad.dimension(0) > 0 && batch_size == (std::size_t) out_grad.dimension(0));
		if (input_layer)
			return typename Base::Data();
		detail::check(cattle_hip_layer_set_input_layer(device.get(), 0));
		typename Base::Data prev_out_grad(detail::batch_dims<typename Base::Dims,Rank>(batch_size, input_dims));
		detail::check(cattle_hip_layer_backward(device.get(), out_grad.data(), CATTLE_HIP_HOST, batch_size,
				prev_out_grad.data(), CATTLE_HIP_HOST));
		return prev_out_grad;
	}
	/** The argmax cache of a max pooling layer, OH*OW rows of channels*batch entries (MaxPoolLayer.hpp:58-62). */
	inline std::vector<unsigned> get_max_indices() const {
		std::vector<unsigned> inds(batch_size * output_dims.get_volume());
		detail::check(cattle_hip_maxpool_indices(device.get(), inds.data(), CATTLE_HIP_HOST));
		return inds;
	}
private:
	inline static typename Base::Dims output_dims_for(const typename Base::Dims& input_dims, std::size_t receptor_height,
			std::size_t receptor_width, std::size_t vertical_stride, std::size_t horizontal_stride) {
		const std::array<std::size_t,3> in = detail::extended<typename Base::Dims,Rank>(input_dims);
		assert(in[0] >= receptor_height && in[1] >= receptor_width);
		std::array<std::size_t,3> out = { { (in[0] - receptor_height) / vertical_stride + 1,
				(in[1] - receptor_width) / horizontal_stride + 1, in[2] } };
		return detail::contracted<typename Base::Dims,Rank>(out);
	}
	inline void create_device_layer() {
		const std::array<std::size_t,3> in = detail::extended<typename Base::Dims,Rank>(input_dims);
		detail::check(cattle_hip_pool_create(detail::ScalarCode<Scalar>::value, Kind, in[0], in[1], in[2], receptor_height,
				receptor_width, vertical_stride, horizontal_stride, device.out()));
	}
	const typename Base::Dims input_dims, output_dims;
	const std::size_t receptor_height, receptor_width, vertical_stride, horizontal_stride;
	bool input_layer;
	std::size_t batch_size;
	detail::Handle device;
};

template<typename Scalar, std::size_t Rank = 3>
class MaxPoolHIPLayer : public PoolHIPLayer<Scalar,Rank,CATTLE_HIP_POOL_MAX> {
public:
	inline MaxPoolHIPLayer(const typename Layer<Scalar,Rank>::Dims& input_dims, std::size_t receptor_height = 2,
			std::size_t receptor_width = 2, std::size_t vertical_stride = 2, std::size_t horizontal_stride = 2) :
				PoolHIPLayer<Scalar,Rank,CATTLE_HIP_POOL_MAX>(input_dims, receptor_height, receptor_width, vertical_stride,
						horizontal_stride) { }
};

template<typename Scalar>
class MaxPoolHIPLayer<Scalar,1> : public PoolHIPLayer<Scalar,1,CATTLE_HIP_POOL_MAX> {
public:
	inline MaxPoolHIPLayer(const typename Layer<Scalar,1>::Dims& input_dims, std::size_t receptor_length = 2,
			std::size_t stride = 2) :
				PoolHIPLayer<Scalar,1,CATTLE_HIP_POOL_MAX>(input_dims, receptor_length, 1, stride, 1) { }
};

template<typename Scalar, std::size_t Rank = 3>
class MeanPoolHIPLayer : public PoolHIPLayer<Scalar,Rank,CATTLE_HIP_POOL_MEAN> {
public:
	inline MeanPoolHIPLayer(const typename Layer<Scalar,Rank>::Dims& input_dims, std::size_t receptor_height = 2,
			std::size_t receptor_width = 2, std::size_t vertical_stride = 2, std::size_t horizontal_stride = 2) :
				PoolHIPLayer<Scalar,Rank,CATTLE_HIP_POOL_MEAN>(input_dims, receptor_height, receptor_width, vertical_stride,
						horizontal_stride) { }
};

template<typename Scalar>
class MeanPoolHIPLayer<Scalar,1> : public PoolHIPLayer<Scalar,1,CATTLE_HIP_POOL_MEAN> {
public:
	inline MeanPoolHIPLayer(const typename Layer<Scalar,1>::Dims& input_dims, std::size_t receptor_length = 2,
			std::size_t stride = 2) :
				PoolHIPLayer<Scalar,1,CATTLE_HIP_POOL_MEAN>(input_dims, receptor_length, 1, stride, 1) { }
};

} /* namespace hip */
} /* namespace cattle */

#endif /* CATTLE_HIP_HIPLAYERS_HPP_ */
