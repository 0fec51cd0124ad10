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

/* Accesses through the pointers of the step structures, told to be global memory: a pointer that sits in a structure is
 * not known to be one, the compiler then emits flat accesses, and those count against the LDS counter as well as the
 * memory counter - inside a GEMM kernel every wait for an LDS read would wait for them too. */
template<typename T>
__device__ __forceinline__ T lstm_ld(const T* p, unsigned i) {
	return ((const __attribute__((address_space(1))) T*) p)[i];
}
template<typename T>
__device__ __forceinline__ void lstm_st(T* p, unsigned i, T v) {
	__builtin_nontemporal_store(v, (__attribute__((address_space(1))) T*) p + i);
}

/* The usual cell: sigmoid gates, tanh on the candidates and on the state. Kernels test for it once and run the
 * arithmetic with the kinds known at compile time (STD): straight-line code whose independent elements the compiler can
 * interleave, where the run-time switch is a chain of branches per activation. */
template<typename T>
__device__ __forceinline__ bool lstm_standard_acts(const LstmActs<T>& a) {
	return a.kind[0] == ACT_SIGMOID && a.kind[1] == ACT_SIGMOID && a.kind[2] == ACT_TANH && a.kind[3] == ACT_TANH &&
			a.kind[4] == ACT_SIGMOID;
}
/* activation WHICH of the cell (0 forget, 1 write, 2 candidate, 3 state, 4 read) */
template<typename T, bool STD, int WHICH>
__device__ __forceinline__ T lstm_act_f(const LstmActs<T>& a, T x) {
	if constexpr (STD)
		return act_f<T, (WHICH == 2 || WHICH == 3) ? ACT_TANH : ACT_SIGMOID>(x, (T) 0);
	else
		return act_f_rt<T>(a.kind[WHICH], x, a.param[WHICH]);
}
template<typename T, bool STD, int WHICH>
__device__ __forceinline__ T lstm_act_b(const LstmActs<T>& a, T x, T y, T g) {
	if constexpr (STD)
		return act_b<T, (WHICH == 2 || WHICH == 3) ? ACT_TANH : ACT_SIGMOID>(x, y, g, (T) 0);
	else
		return act_b_rt<T>(a.kind[WHICH], x, y, g, a.param[WHICH]);
}

/* Offset of element (n, rest) of time step t in a sequence tensor (N, T_len, ...): element e = n + N * rest of a
 * step's slab. A slab of P elements is a whole number of samples, so gate g of element e is (n, rest + g * P / N):
 * one 32-bit division per element serves all of its accesses. All offsets are formed in 32 bits: the host checks that
 * four slabs, and every sequence tensor, stay below 2^31 elements. */
__device__ __forceinline__ unsigned seq_offset(unsigned n, unsigned rest, int N, int T_len, int t) {
	return n + (unsigned) N * ((unsigned) t + (unsigned) T_len * rest);
}

/* Column of the weight matrix [forget | write | candidate | read] (hidden columns each) that sits at column f of the
 * layout whose groups of 4 cb columns hold the four gates of cb hidden channels: gate (f / cb) % 4 of channel
 * (f / (4 cb)) cb + f % cb. */
__host__ __device__ __forceinline__ int lstm_gate_column(int f, int cb, int hidden) {
	return ((f / cb) & 3) * hidden + (f / (4 * cb)) * cb + f % cb;
}

/* What the forward step of an element reads besides the weighted previous output. */
template<typename T> struct LstmForwardInputs { T zx[4]; T prev; };

template<typename T>
__device__ __forceinline__ LstmForwardInputs<T> lstm_forward_load(const LstmForwardStep<T>& A, unsigned e) {
	const unsigned N = (unsigned) A.N, slab_rows = (unsigned) A.P / N;
	const unsigned rest = e / N, n = e - rest * N;
	LstmForwardInputs<T> in;
	#pragma unroll
	for (int g = 0; g < 4; ++g)
		in.zx[g] = A.zx ? lstm_ld<T>(A.zx, seq_offset(n, rest + g * slab_rows, A.N, A.zx_T, A.zx_t)) : (T) 0;
	in.prev = A.prev_state ? lstm_ld<T>(A.prev_state, e) : (T) 0;
	return in;
}

/* What the forward step of an element writes: the gates' pre-activation values and values, the state, the activated
 * state and the hidden output. */
template<typename T> struct LstmForwardOutputs { T v[4], y[4], s, as, h; };

/* The arithmetic of the forward step, registers only. zh4: the weighted previous output of the element's four gates
 * (bias included) if has_zh; there is none at the first step. (An array and a flag, not a pointer that may be null: the
 * array behind such a pointer cannot stay in registers.) */
template<typename T, bool STD = false>
__device__ __forceinline__ LstmForwardOutputs<T> lstm_forward_compute(const LstmForwardStep<T>& A, const LstmForwardInputs<T>& in,
		bool has_zh, const T (&zh4)[4]) {
	LstmForwardOutputs<T> o;
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		/* weighted input + weighted previous output (:312, :327, :342, :373), their product with multiplicative
		 * integration (:303-311); a step with only one of the two takes it as it is */
		T v = in.zx[g];
		if (has_zh)
			v = A.zx ? (A.mul_int ? v * zh4[g] : v + zh4[g]) : zh4[g];
		o.v[g] = v;
	}
	o.y[0] = lstm_act_f<T, STD, 0>(A.a, o.v[0]);
	o.y[1] = lstm_act_f<T, STD, 1>(A.a, o.v[1]);
	o.y[2] = lstm_act_f<T, STD, 2>(A.a, o.v[2]);
	o.y[3] = lstm_act_f<T, STD, 4>(A.a, o.v[3]);                /* the fourth gate is the read filter */
	o.s = o.y[0] * in.prev;                                     /* selective remembrance (:314) */
	o.s += o.y[1] * o.y[2];                                     /* write filter * candidates (:345) */
	o.as = lstm_act_f<T, STD, 3>(A.a, o.s);
	o.h = o.y[3] * o.as;                                        /* read filter * activated state (:383) */
	return o;
}

template<typename T>
__device__ __forceinline__ void lstm_forward_store(const LstmForwardStep<T>& A, unsigned e, const LstmForwardOutputs<T>& o) {
	const unsigned N = (unsigned) A.N, P = (unsigned) A.P;
	const unsigned rest = e / N, n = e - rest * N;
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		if (A.z)
			lstm_st<T>(A.z, (unsigned) g * P + e, o.v[g]);
		lstm_st<T>(A.gates, (unsigned) g * P + e, o.y[g]);
	}
	lstm_st<T>(A.state, e, o.s);
	lstm_st<T>(A.act_state, e, o.as);
	if (A.hprev_all) {
		if (A.h_t < A.h_T)
			lstm_st<T>(A.hprev_all, seq_offset(n, rest, A.N, A.h_T, A.h_t), o.h);
		if (!A.prev_state)                                      /* first step: no previous output, slab 0 is zero */
			lstm_st<T>(A.hprev_all, seq_offset(n, rest, A.N, A.h_T, 0), (T) 0);
	}
	if (A.out)
		lstm_st<T>(A.out, seq_offset(n, rest, A.N, A.out_T, A.out_t), o.h);
}

/* The same for V consecutive elements e0 .. e0 + V - 1 (e0 and N multiples of V, so they are V consecutive samples of
 * one place and consecutive in every tensor of the step; tensors aligned to V elements): one access of V elements per
 * tensor instead of V accesses, and the index arithmetic once. */
template<typename T, int V>
__device__ __forceinline__ void lstm_ldv(T (&dst)[V], const T* p, unsigned i) {
	if constexpr (V == 1) {
		dst[0] = lstm_ld<T>(p, i);
	} else {
		typedef T vt __attribute__((ext_vector_type(V)));
		const vt v = *(const __attribute__((address_space(1))) vt*) (p + i);
		#pragma unroll
		for (int k = 0; k < V; ++k)
			dst[k] = v[k];
	}
}
template<typename T, int V>
__device__ __forceinline__ void lstm_stv(T* p, unsigned i, const T (&src)[V]) {
	if constexpr (V == 1) {
		lstm_st<T>(p, i, src[0]);
	} else {
		typedef T vt __attribute__((ext_vector_type(V)));
		vt v;
		#pragma unroll
		for (int k = 0; k < V; ++k)
			v[k] = src[k];
		__builtin_nontemporal_store(v, (__attribute__((address_space(1))) vt*) (p + i));
	}
}
template<typename T, int V>
__device__ __forceinline__ void lstm_forward_load_vec(const LstmForwardStep<T>& A, unsigned e0, LstmForwardInputs<T> (&in)[V]) {
	const unsigned N = (unsigned) A.N, slab_rows = (unsigned) A.P / N;
	const unsigned rest = e0 / N, n = e0 - rest * N;
	T v[V];
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		if (A.zx)
			lstm_ldv<T, V>(v, A.zx, seq_offset(n, rest + g * slab_rows, A.N, A.zx_T, A.zx_t));
		#pragma unroll
		for (int k = 0; k < V; ++k)
			in[k].zx[g] = A.zx ? v[k] : (T) 0;
	}
	if (A.prev_state)
		lstm_ldv<T, V>(v, A.prev_state, e0);
	#pragma unroll
	for (int k = 0; k < V; ++k)
		in[k].prev = A.prev_state ? v[k] : (T) 0;
}
template<typename T, int V>
__device__ __forceinline__ void lstm_forward_store_vec(const LstmForwardStep<T>& A, unsigned e0, const LstmForwardOutputs<T> (&o)[V]) {
	const unsigned N = (unsigned) A.N, P = (unsigned) A.P;
	const unsigned rest = e0 / N, n = e0 - rest * N;
	T v[V];
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		if (A.z) {
			#pragma unroll
			for (int k = 0; k < V; ++k)
				v[k] = o[k].v[g];
			lstm_stv<T, V>(A.z, (unsigned) g * P + e0, v);
		}
		#pragma unroll
		for (int k = 0; k < V; ++k)
			v[k] = o[k].y[g];
		lstm_stv<T, V>(A.gates, (unsigned) g * P + e0, v);
	}
	#pragma unroll
	for (int k = 0; k < V; ++k)
		v[k] = o[k].s;
	lstm_stv<T, V>(A.state, e0, v);
	#pragma unroll
	for (int k = 0; k < V; ++k)
		v[k] = o[k].as;
	lstm_stv<T, V>(A.act_state, e0, v);
	#pragma unroll
	for (int k = 0; k < V; ++k)
		v[k] = o[k].h;
	if (A.hprev_all) {
		if (A.h_t < A.h_T)
			lstm_stv<T, V>(A.hprev_all, seq_offset(n, rest, A.N, A.h_T, A.h_t), v);
		if (!A.prev_state) {                                    /* first step: no previous output, slab 0 is zero */
			T zero[V];
			#pragma unroll
			for (int k = 0; k < V; ++k)
				zero[k] = (T) 0;
			lstm_stv<T, V>(A.hprev_all, seq_offset(n, rest, A.N, A.h_T, 0), zero);
		}
	}
	if (A.out)
		lstm_stv<T, V>(A.out, seq_offset(n, rest, A.N, A.out_T, A.out_t), v);
}
/* Whether the step's tensors allow accesses of V elements. */
template<typename T>
inline bool lstm_forward_vectors(const LstmForwardStep<T>& A, int V) {
	const uintptr_t mask = (uintptr_t) V * sizeof(T) - 1;
	const void* const ptrs[8] = { A.zx, A.prev_state, A.z, A.gates, A.state, A.act_state, A.hprev_all, A.out };
	for (const void* q : ptrs)
		if ((reinterpret_cast<uintptr_t>(q) & mask) != 0)
			return false;
	return A.N % V == 0 && A.P % (size_t) V == 0;
}

/* Every load of the element comes before its first store: the tensors are not declared free of aliases, and a store
 * between two loads would make the second wait for the first. */
template<typename T, bool STD = false>
__device__ __forceinline__ void lstm_forward_element(const LstmForwardStep<T>& A, unsigned e, bool has_zh, const T (&zh4)[4]) {
	const LstmForwardInputs<T> in = lstm_forward_load<T>(A, e);
	lstm_forward_store<T>(A, e, lstm_forward_compute<T, STD>(A, in, has_zh, zh4));
}

/* What the backward step of element e reads, for the usual cell (no kept pre-activation values, no multiplicative
 * integration): a kernel that knows its elements early can fetch these before its own work and run the step on them later
 * (lstm_backward_finish), instead of paying a round trip to memory at its end. */
template<typename T>
struct LstmBackwardInputs {
	T og, gates[4], as, sgrad, state, prev;
};
template<typename T>
__device__ __forceinline__ bool lstm_backward_can_preload(const LstmBackwardStep<T>& A) {
	return A.z == nullptr && A.zx_fwd == nullptr;
}
template<typename T>
__device__ __forceinline__ LstmBackwardInputs<T> lstm_backward_load(const LstmBackwardStep<T>& A, unsigned e, bool has_dh) {
	const unsigned N = (unsigned) A.N, P = (unsigned) A.P;
	const unsigned rest = e / N, n = e - rest * N;
	LstmBackwardInputs<T> in;
	in.og = A.out_grad ? lstm_ld<T>(A.out_grad, seq_offset(n, rest, A.N, A.og_T, A.og_t)) : (T) 0;
	#pragma unroll
	for (int g = 0; g < 4; ++g)
		in.gates[g] = lstm_ld<T>(A.gates, (unsigned) g * P + e);
	in.as = lstm_ld<T>(A.act_state, e);
	in.sgrad = has_dh ? lstm_ld<T>(A.state_grad, e) : (T) 0;
	in.state = lstm_ld<T>(A.state, e);
	in.prev = A.prev_state ? lstm_ld<T>(A.prev_state, e) : (T) 0;
	return in;
}
/* The step itself on preloaded inputs: the same arithmetic, in the same order, as lstm_backward_element below. */
template<typename T, bool STD = false>
__device__ __forceinline__ void lstm_backward_finish(const LstmBackwardStep<T>& A, unsigned e, bool has_dh, T dh,
		const LstmBackwardInputs<T>& in) {
	const unsigned N = (unsigned) A.N, P = (unsigned) A.P;
	const unsigned slab_rows = P / N;
	const unsigned rest = e / N, n = e - rest * N;
	T hg = has_dh ? dh : (T) 0;
	if (A.out_grad)
		hg += in.og;
	const T f = in.gates[0], w = in.gates[1], c = in.gates[2], r = in.gates[3];
	const T as = in.as;
	const T sg = in.sgrad + lstm_act_b<T, STD, 3>(A.a, in.state, as, r * hg);
	T d[4];
	d[3] = lstm_act_b<T, STD, 4>(A.a, (T) 0, r, as * hg);
	d[2] = lstm_act_b<T, STD, 2>(A.a, (T) 0, c, w * sg);
	d[1] = lstm_act_b<T, STD, 1>(A.a, (T) 0, w, c * sg);
	d[0] = lstm_act_b<T, STD, 0>(A.a, (T) 0, f, in.prev * sg);
	lstm_st<T>(A.state_grad, e, sg * f);
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		if (A.dzx_all)
			lstm_st<T>(A.dzx_all, seq_offset(n, rest + g * slab_rows, A.N, A.x_T, A.x_t), d[g]);
		if (A.dzh_all)
			lstm_st<T>(A.dzh_all, seq_offset(n, rest + g * slab_rows, A.N, A.h_T, A.h_t), A.prev_state ? d[g] : (T) 0);
	}
}

/* Backward step of element e. dh: the gradient of the element's hidden output that came back through the next
 * step's output-side kernels; has_dh is false at the last time step, where there is none and the state gradient
 * starts at zero (:422-425). */
template<typename T, bool STD = false>
__device__ __forceinline__ void lstm_backward_element(const LstmBackwardStep<T>& A, unsigned e, bool has_dh, T dh) {
	const unsigned N = (unsigned) A.N, P = (unsigned) A.P;
	const unsigned slab_rows = P / N;
	const unsigned rest = e / N, n = e - rest * N;
	T hg = has_dh ? dh : (T) 0;
	if (A.out_grad)
		hg += lstm_ld<T>(A.out_grad, seq_offset(n, rest, A.N, A.og_T, A.og_t));       /* :431-438 */
	const T f = lstm_ld<T>(A.gates, e), w = lstm_ld<T>(A.gates, P + e), c = lstm_ld<T>(A.gates, 2u * P + e), r = lstm_ld<T>(A.gates, 3u * P + e);
	const T as = lstm_ld<T>(A.act_state, e);
	const T sg = (has_dh ? lstm_ld<T>(A.state_grad, e) : (T) 0) + lstm_act_b<T, STD, 3>(A.a, lstm_ld<T>(A.state, e), as, r * hg);      /* :440 */
	T zin[4] = { (T) 0, (T) 0, (T) 0, (T) 0 };
	if (A.z) {
		#pragma unroll
		for (int g = 0; g < 4; ++g)
			zin[g] = lstm_ld<T>(A.z, (unsigned) g * P + e);
	}
	T d[4];
	d[3] = lstm_act_b<T, STD, 4>(A.a, zin[3], r, as * hg);                       /* :441 */
	d[2] = lstm_act_b<T, STD, 2>(A.a, zin[2], c, w * sg);                        /* :442 */
	d[1] = lstm_act_b<T, STD, 1>(A.a, zin[1], w, c * sg);                            /* :443 */
	d[0] = lstm_act_b<T, STD, 0>(A.a, zin[0], f, (A.prev_state ? lstm_ld<T>(A.prev_state, e) : (T) 0) * sg);  /* :444 */
	/* multiplicative integration at a step with both an input and a previous output (zx_fwd and zh_fwd are that
	 * step's weighted input and weighted output): each side's gradient carries the other side (:449-466) */
	T to_input[4], to_output[4];
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		to_input[g] = to_output[g] = d[g];
		if (A.zx_fwd) {
			to_input[g] = lstm_ld<T>(A.zh_fwd, (unsigned) g * P + e) * d[g];
			to_output[g] = lstm_ld<T>(A.zx_fwd, seq_offset(n, rest + g * slab_rows, A.N, A.x_T, A.x_t)) * d[g];
		}
	}
	lstm_st<T>(A.state_grad, e, sg * f);                                                                                  /* :445 */
	#pragma unroll
	for (int g = 0; g < 4; ++g) {
		if (A.dzx_all)
			lstm_st<T>(A.dzx_all, seq_offset(n, rest + g * slab_rows, A.N, A.x_T, A.x_t), to_input[g]);
		/* what the output-side kernels' pass_back receives; step 0 has no previous output to pair with: its slab is zero */
		if (A.dzh_all)
			lstm_st<T>(A.dzh_all, seq_offset(n, rest + g * slab_rows, A.N, A.h_T, A.h_t), A.prev_state ? to_output[g] : (T) 0);
	}
}

} /* namespace cattle_hip */

#endif
