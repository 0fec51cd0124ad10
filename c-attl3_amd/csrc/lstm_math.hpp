/*
 * lstm_math.hpp — the element-wise part of an LSTM cell step (neural_network/LSTMNeuralNetwork.hpp:283-394 forward,
 * :436-466 backward) as device functions of one state element, shared by the streaming kernels
 * (pointwise_kernels.hip) and by the GEMM kernels that apply it to their own results (gemm_kernels.hip).
 *
 * The four gates (forget, write, candidate, read) are the channel blocks of one tensor, so gate g of element e sits
 * at g*P + e in a per-step tensor. Tensors that span all time steps are (N, T, ...) column-major: element e of step t
 * is at n + N*(t + T*rest) with n = e % N, rest = e / N.
 */
#ifndef CATTLE_HIP_LSTM_MATH_HPP_
#define CATTLE_HIP_LSTM_MATH_HPP_

#include "common.hpp"
#include "act_math.hpp"

namespace cattle_hip {

template<typename T>
__device__ __forceinline__ T act_f_rt(int kind, T x, T p) {
	switch (kind) {
	case ACT_IDENTITY: return act_f<T, ACT_IDENTITY>(x, p);
	case ACT_SCALED: return act_f<T, ACT_SCALED>(x, p);
	case ACT_BINARY_STEP: return act_f<T, ACT_BINARY_STEP>(x, p);
	case ACT_SIGMOID: return act_f<T, ACT_SIGMOID>(x, p);
	case ACT_TANH: return act_f<T, ACT_TANH>(x, p);
	case ACT_SOFTSIGN: return act_f<T, ACT_SOFTSIGN>(x, p);
	case ACT_SOFTPLUS: return act_f<T, ACT_SOFTPLUS>(x, p);
	case ACT_RELU: return act_f<T, ACT_RELU>(x, p);
	case ACT_LEAKY_RELU: return act_f<T, ACT_LEAKY_RELU>(x, p);
	case ACT_ELU: return act_f<T, ACT_ELU>(x, p);
	default: return act_f<T, ACT_SWISH>(x, p);
	}
}

template<typename T>
__device__ __forceinline__ T act_b_rt(int kind, T x, T y, T g, T p) {
	switch (kind) {
	case ACT_IDENTITY: return act_b<T, ACT_IDENTITY>(x, y, g, p);
	case ACT_SCALED: return act_b<T, ACT_SCALED>(x, y, g, p);
	case ACT_BINARY_STEP: return act_b<T, ACT_BINARY_STEP>(x, y, g, p);
	case ACT_SIGMOID: return act_b<T, ACT_SIGMOID>(x, y, g, p);
	case ACT_TANH: return act_b<T, ACT_TANH>(x, y, g, p);
	case ACT_SOFTSIGN: return act_b<T, ACT_SOFTSIGN>(x, y, g, p);
	case ACT_SOFTPLUS: return act_b<T, ACT_SOFTPLUS>(x, y, g, p);
	case ACT_RELU: return act_b<T, ACT_RELU>(x, y, g, p);
	case ACT_LEAKY_RELU: return act_b<T, ACT_LEAKY_RELU>(x, y, g, p);
	case ACT_ELU: return act_b<T, ACT_ELU>(x, y, g, p);
	default: return act_b<T, ACT_SWISH>(x, y, g, p);
	}
}

/* Offset of element (n, rest) of time step t in a sequence tensor (N, T_len, ...): element e = n + N * rest of a
 * step's slab. A slab of P elements is a whole number of samples, so gate g of element e is (n, rest + g * P / N):
 * one 32-bit division per element serves all of its accesses (the host checks that 4 P fits 32 bits). */
__device__ __forceinline__ size_t seq_offset(unsigned n, unsigned rest, int N, int T_len, int t) {
	return n + (size_t) N * ((size_t) t + (size_t) T_len * rest);
}

/* Forward step of element e. zh4: the weighted previous output of the element's four gates (bias included), or null
 * at the first step. */
template<typename T>
__device__ __forceinline__ void lstm_forward_element(const LstmForwardStep<T>& A, unsigned e, const T* zh4) {
	const unsigned N = (unsigned) A.N, P = (unsigned) A.P;
	const unsigned slab_rows = P / N;
	const unsigned rest = e / N, n = e - rest * N;
	/* every load of the element before its first store: the tensors are not declared free of aliases, and a store
	 * between two loads would make the second wait for the first */
	T v[4], y[4];
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		/* weighted input + weighted previous output (:312, :327, :342, :373), their product with multiplicative
		 * integration (:303-311); a step with only one of the two takes it as it is */
		v[g] = (T) 0;
		if (A.zx)
			v[g] = A.zx[seq_offset(n, rest + g * slab_rows, A.N, A.zx_T, A.zx_t)];
		if (zh4)
			v[g] = A.zx ? (A.mul_int ? v[g] * zh4[g] : v[g] + zh4[g]) : zh4[g];
	}
	const T prev = A.prev_state ? A.prev_state[e] : (T) 0;
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		if (A.z)
			A.z[(size_t) g * P + e] = v[g];
		const int which = g < 3 ? g : 4;                        /* kinds: forget, write, candidate, state, read */
		y[g] = act_f_rt<T>(A.a.kind[which], v[g], A.a.param[which]);
		A.gates[(size_t) g * P + e] = y[g];
	}
	T s = y[0] * prev;                                          /* selective remembrance (:314) */
	s += y[1] * y[2];                                           /* write filter * candidates (:345) */
	A.state[e] = s;
	const T as = act_f_rt<T>(A.a.kind[3], s, A.a.param[3]);
	A.act_state[e] = as;
	const T h = y[3] * as;                                      /* read filter * activated state (:383) */
	if (A.hprev_all) {
		if (A.h_t < A.h_T)
			A.hprev_all[seq_offset(n, rest, A.N, A.h_T, A.h_t)] = h;
		if (!A.prev_state)                                      /* first step: no previous output, slab 0 is zero */
			A.hprev_all[seq_offset(n, rest, A.N, A.h_T, 0)] = (T) 0;
	}
	if (A.out)
		A.out[seq_offset(n, rest, A.N, A.out_T, A.out_t)] = h;
}

/* Backward step of element e. dh: the gradient of the element's hidden output that came back through the next
 * step's output-side kernels; has_dh is false at the last time step, where there is none and the state gradient
 * starts at zero (:422-425). */
template<typename T>
__device__ __forceinline__ void lstm_backward_element(const LstmBackwardStep<T>& A, unsigned e, bool has_dh, T dh) {
	const unsigned N = (unsigned) A.N, P = (unsigned) A.P;
	const unsigned slab_rows = P / N;
	const unsigned rest = e / N, n = e - rest * N;
	T hg = has_dh ? dh : (T) 0;
	if (A.out_grad)
		hg += A.out_grad[seq_offset(n, rest, A.N, A.og_T, A.og_t)];       /* :431-438 */
	const T f = A.gates[e], w = A.gates[(size_t) P + e], c = A.gates[(size_t) 2 * P + e], r = A.gates[(size_t) 3 * P + e];
	const T as = A.act_state[e];
	const T sg = (has_dh ? A.state_grad[e] : (T) 0) + act_b_rt<T>(A.a.kind[3], A.state[e], as, r * hg, A.a.param[3]);      /* :440 */
	T zin[4] = { (T) 0, (T) 0, (T) 0, (T) 0 };
	if (A.z) {
		#pragma unroll
		for (int g = 0; g < 4; ++g)
			zin[g] = A.z[(size_t) g * P + e];
	}
	T d[4];
	d[3] = act_b_rt<T>(A.a.kind[4], zin[3], r, as * hg, A.a.param[4]);                       /* :441 */
	d[2] = act_b_rt<T>(A.a.kind[2], zin[2], c, w * sg, A.a.param[2]);                        /* :442 */
	d[1] = act_b_rt<T>(A.a.kind[1], zin[1], w, c * sg, A.a.param[1]);                            /* :443 */
	d[0] = act_b_rt<T>(A.a.kind[0], zin[0], f, (A.prev_state ? A.prev_state[e] : (T) 0) * sg, A.a.param[0]);  /* :444 */
	/* multiplicative integration at a step with both an input and a previous output (zx_fwd and zh_fwd are that
	 * step's weighted input and weighted output): each side's gradient carries the other side (:449-466) */
	T to_input[4], to_output[4];
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		to_input[g] = to_output[g] = d[g];
		if (A.zx_fwd) {
			to_input[g] = A.zh_fwd[(size_t) g * P + e] * d[g];
			to_output[g] = A.zx_fwd[seq_offset(n, rest + g * slab_rows, A.N, A.x_T, A.x_t)] * d[g];
		}
	}
	A.state_grad[e] = sg * f;                                                                                  /* :445 */
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		if (A.dzx_all)
			A.dzx_all[seq_offset(n, rest + g * slab_rows, A.N, A.x_T, A.x_t)] = to_input[g];
		/* what the output-side kernels' pass_back receives; step 0 has no previous output to pair with: its slab is zero */
		if (A.dzh_all)
			A.dzh_all[seq_offset(n, rest + g * slab_rows, A.N, A.h_T, A.h_t)] = A.prev_state ? to_output[g] : (T) 0;
	}
}

} /* namespace cattle_hip */

#endif
