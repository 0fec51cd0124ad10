/*
 * act_math.hpp — the element-wise activation functions of layer/activation/ as device functions, shared by the
 * streaming kernels (pointwise_kernels.hip) and the GEMM epilogues and operand loads (gemm_kernels.hip).
 */
#ifndef CATTLE_HIP_ACT_MATH_HPP_
#define CATTLE_HIP_ACT_MATH_HPP_

#include <hip/hip_runtime.h>
#include <type_traits>

namespace cattle_hip {

enum ActKind {
	ACT_IDENTITY = 0, ACT_SCALED = 1, ACT_BINARY_STEP = 2, ACT_SIGMOID = 3, ACT_TANH = 4, ACT_SOFTSIGN = 5,
	ACT_SOFTPLUS = 6, ACT_RELU = 7, ACT_LEAKY_RELU = 8, ACT_ELU = 9, ACT_SWISH = 10
};

__device__ __forceinline__ float dev_exp(float v) { return expf(v); }
__device__ __forceinline__ double dev_exp(double v) { return exp(v); }
__device__ __forceinline__ float dev_log(float v) { return logf(v); }
__device__ __forceinline__ double dev_log(double v) { return log(v); }
__device__ __forceinline__ float dev_tanh(float v) { return tanhf(v); }
__device__ __forceinline__ double dev_tanh(double v) { return tanh(v); }
__device__ __forceinline__ float dev_sqrt(float v) { return sqrtf(v); }
__device__ __forceinline__ double dev_sqrt(double v) { return sqrt(v); }

/* Forward functions; each cites the reference layer whose formula it evaluates. */
template<typename T, int KIND>
__device__ __forceinline__ T act_f(T x, T p) {
	switch (KIND) {
	case ACT_IDENTITY: return x;                                        /* IdentityActivationLayer.hpp:37-42 */
	case ACT_SCALED: return x * p;                                      /* ScaledActivationLayer.hpp:38-43 */
	case ACT_BINARY_STEP: return (T) (x >= (T) 0);                      /* BinaryStepActivationLayer.hpp:42-47 */
	case ACT_SIGMOID: return (T) 1 / (dev_exp(-x) + (T) 1);             /* SigmoidActivationLayer.hpp:38-43 */
	case ACT_TANH: return dev_tanh(x);                                  /* TanhActivationLayer.hpp:38-43 */
	case ACT_SOFTSIGN: return x / ((T) 1 + (x < (T) 0 ? -x : x));       /* SoftsignActivationLayer.hpp:39-44 */
	case ACT_SOFTPLUS: return dev_log(dev_exp(x) + (T) 1);              /* SoftplusActivationLayer.hpp:40-45 */
	case ACT_RELU: return x > (T) 0 ? x : (x == x ? (T) 0 : x);         /* ReLUActivationLayer.hpp:45-50 */
	case ACT_LEAKY_RELU: { const T ax = x * p; return x > ax ? x : (ax == ax ? ax : x); }   /* LeakyReLU :50-55 */
	case ACT_ELU: return x >= (T) 0 ? x : p * (dev_exp(x) - (T) 1);     /* ELUActivationLayer.hpp:55-64 */
	case ACT_SWISH: return x * ((T) 1 / (dev_exp(-p * x) + (T) 1));     /* SwishActivationLayer.hpp:45-51 */
	}
	return x;
}

/* Backward functions of (input x, output y, upstream gradient g). */
template<typename T, int KIND>
__device__ __forceinline__ T act_b(T x, T y, T g, T p) {
	switch (KIND) {
	case ACT_IDENTITY: return g;                                        /* IdentityActivationLayer.hpp:43-49 */
	case ACT_SCALED: return g * p;                                      /* ScaledActivationLayer.hpp:44-50 */
	case ACT_BINARY_STEP: return (T) 0;                                 /* BinaryStepActivationLayer.hpp:48-54 */
	case ACT_SIGMOID: return (y * ((T) 1 - y)) * g;                     /* SigmoidActivationLayer.hpp:44-50 */
	case ACT_TANH: return ((T) 1 - y * y) * g;                          /* TanhActivationLayer.hpp:44-50 */
	case ACT_SOFTSIGN: { const T d = (T) 1 + (x < (T) 0 ? -x : x); return ((T) 1 / (d * d)) * g; }   /* :45-51 */
	case ACT_SOFTPLUS: return ((T) 1 / (dev_exp(-x) + (T) 1)) * g;      /* SoftplusActivationLayer.hpp:46-52 */
	case ACT_RELU: return (T) (x >= (T) 0) * g;                         /* ReLUActivationLayer.hpp:51-57 */
	case ACT_LEAKY_RELU: return (x >= (T) 0 ? (T) 1 : p) * g;           /* LeakyReLUActivationLayer.hpp:56-62 */
	case ACT_ELU: return (x >= (T) 0 ? (T) 1 : (y + p)) * g;            /* ELUActivationLayer.hpp:65-78 */
	case ACT_SWISH: {                                                   /* SwishActivationLayer.hpp:52-59 */
		const T s = (T) 1 / (dev_exp(-p * x) + (T) 1);
		return s * ((((T) 1 - s) * p) * x + (T) 1) * g;
	}
	}
	return g;
}

/* Which cached operands the backward of a kind actually reads (the others may be null). */
__host__ __device__ constexpr bool act_needs_x(int k) {
	return k == ACT_SOFTSIGN || k == ACT_SOFTPLUS || k == ACT_RELU || k == ACT_LEAKY_RELU || k == ACT_ELU || k == ACT_SWISH;
}
__host__ __device__ constexpr bool act_needs_y(int k) {
	return k == ACT_SIGMOID || k == ACT_TANH || k == ACT_ELU;
}


/* ---- activations applied inside a GEMM epilogue -------------------------------------------------------------------
 * A fused kernel layer does not keep its pre-activation values, so the backward pass must work from the output alone.
 * Sigmoid and tanh already do. For the rectifier family the derivative depends on the sign of the input
 * (x >= 0 ? 1 : slope), which the output loses where it is zero; the fused forward pass therefore stores the output
 * with the sign bit of the input's side: +|y| for x >= 0 (x = -0 counts as 0, as in the reference's x >= 0) and -|y|
 * for x < 0. Numerically nothing changes (-0 equals 0 in every comparison and sum downstream, including the strict
 * '>' of max pooling), and the backward pass reads the side from the sign bit. Valid whenever the function maps
 * negative inputs to non-positive outputs: ReLU, LeakyReLU and ELU with alpha >= 0. The other kinds (softsign,
 * softplus, swish, negative alphas) need the input itself: the epilogue stores it beside the output. */
__host__ __device__ constexpr bool act_sign_coded(int k) {
	return k == ACT_RELU || k == ACT_LEAKY_RELU || k == ACT_ELU;
}
/* whether the backward pass of a fused layer can work from the (sign-coded) output alone */
inline bool act_backward_from_output(int k, double p) {
	if (k == ACT_LEAKY_RELU || k == ACT_ELU)
		return p >= 0;
	return k == ACT_IDENTITY || k == ACT_SCALED || k == ACT_BINARY_STEP || k == ACT_SIGMOID || k == ACT_TANH || k == ACT_RELU;
}

__device__ __forceinline__ bool sign_bit(float v) { return (__float_as_uint(v) >> 31) != 0u; }
__device__ __forceinline__ bool sign_bit(double v) { return (__double_as_longlong(v) < 0); }
__device__ __forceinline__ float with_sign(float mag, bool negative) {
	return __uint_as_float((__float_as_uint(mag) & 0x7fffffffu) | (negative ? 0x80000000u : 0u));
}
__device__ __forceinline__ double with_sign(double mag, bool negative) {
	return __longlong_as_double((__double_as_longlong(mag) & 0x7fffffffffffffffll) | (negative ? (long long) 0x8000000000000000ull : 0ll));
}

/* forward value as a fused epilogue stores it */
template<typename T, int KIND>
__device__ __forceinline__ T act_f_coded(T x, T p) {
	const T y = act_f<T, KIND>(x, p);
	if (act_sign_coded(KIND) && (KIND == ACT_RELU || p >= (T) 0))     /* a negative slope puts positive outputs on both sides */
		return y == y ? with_sign(y, !(x >= (T) 0)) : y;
	return y;
}

/* backward from the coded output y (kinds for which act_backward_from_output holds) */
template<typename T, int KIND>
__device__ __forceinline__ T act_b_coded(T y, T g, T p) {
	switch (KIND) {
	case ACT_RELU: return (T) (!sign_bit(y)) * g;
	case ACT_LEAKY_RELU: return (sign_bit(y) ? p : (T) 1) * g;
	case ACT_ELU: return (sign_bit(y) ? (y + p) : (T) 1) * g;
	default: break;
	}
	return act_b<T, KIND>((T) 0, y, g, p);
}

/* Calls fn(std::integral_constant<int, KIND>) for the run-time kind: the switch sits outside the unrolled loops of a
 * kernel, so each loop body is compiled for one kind. */
template<typename Fn>
__device__ __forceinline__ void act_dispatch(int kind, Fn fn) {
	switch (kind) {
	case ACT_SCALED: fn(std::integral_constant<int, ACT_SCALED>()); break;
	case ACT_BINARY_STEP: fn(std::integral_constant<int, ACT_BINARY_STEP>()); break;
	case ACT_SIGMOID: fn(std::integral_constant<int, ACT_SIGMOID>()); break;
	case ACT_TANH: fn(std::integral_constant<int, ACT_TANH>()); break;
	case ACT_SOFTSIGN: fn(std::integral_constant<int, ACT_SOFTSIGN>()); break;
	case ACT_SOFTPLUS: fn(std::integral_constant<int, ACT_SOFTPLUS>()); break;
	case ACT_RELU: fn(std::integral_constant<int, ACT_RELU>()); break;
	case ACT_LEAKY_RELU: fn(std::integral_constant<int, ACT_LEAKY_RELU>()); break;
	case ACT_ELU: fn(std::integral_constant<int, ACT_ELU>()); break;
	case ACT_SWISH: fn(std::integral_constant<int, ACT_SWISH>()); break;
	default: fn(std::integral_constant<int, ACT_IDENTITY>()); break;
	}
}

} /* namespace cattle_hip */

#endif /* CATTLE_HIP_ACT_MATH_HPP_ */
