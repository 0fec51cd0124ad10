/*
 * train_kernels.hip — the two ends of a training step around the layer stack (gfx950):
 * loss functions with their gradients, and in-place optimizer updates of device-resident
 * parameters. All of it is HBM-bound element-wise or row-reduction work.
 *
 * Batches are the reference's column-major tensors: a non-sequential batch is an N x V matrix
 * (sample n, element j at n + N*j); a sequential batch (N, T, ...) puts time step t of sample n,
 * element j at n + N*(t + T*j). Losses treat every time step as its own N x V problem
 * (loss/UniversalLoss.hpp:89-125), so one kernel covers both with a column stride of N*T.
 */
#include "common.hpp"

#include <limits>

namespace cattle_hip {

namespace {

__device__ __forceinline__ float dev_exp(float v) { return expf(v); }
__device__ __forceinline__ double dev_exp(double v) { return exp(v); }
__device__ __forceinline__ float dev_log(float v) { return logf(v); }
__device__ __forceinline__ double dev_log(double v) { return log(v); }
__device__ __forceinline__ float dev_sqrt(float v) { return sqrtf(v); }
__device__ __forceinline__ double dev_sqrt(double v) { return sqrt(v); }

/* Block shape of the row-reduction kernels: ROWS samples side by side (coalesced along n), each
 * reduced by PARTS threads that stride over the sample's elements. */
constexpr int ROWS = 32, PARTS = 8;

/* Combines the PARTS partial values of each row in a fixed order; every thread of the row gets
 * the result. `lds` holds PARTS * ROWS values. */
template<typename T, bool MAX>
__device__ __forceinline__ T row_combine(T v, T* lds) {
	const int r = threadIdx.x, p = threadIdx.y;
	__syncthreads();
	lds[p * ROWS + r] = v;
	__syncthreads();
	T acc = lds[r];
	#pragma unroll
	for (int q = 1; q < PARTS; ++q) {
		const T e = lds[q * ROWS + r];
		acc = MAX ? (e > acc ? e : acc) : acc + e;
	}
	return acc;
}

template<typename T> struct MachineEps;
template<> struct MachineEps<float> { static constexpr float value = 1.1920928955078125e-07f; };
template<> struct MachineEps<double> { static constexpr double value = 2.220446049250313e-16; };

__device__ __forceinline__ float dev_abs(float v) { return fabsf(v); }
__device__ __forceinline__ double dev_abs(double v) { return fabs(v); }

/* NumericUtils::almost_equal with its default epsilons (core/NumericUtils.hpp:42-49) */
template<typename T>
__device__ __forceinline__ bool almost_equal(T a, T b) {
	const T e = MachineEps<T>::value;
	const T diff = dev_abs(a - b);
	if (diff <= e)
		return true;
	const T aa = dev_abs(a), ab = dev_abs(b);
	return diff <= (aa > ab ? aa : ab) * e;
}

/* NumericUtils::decidedly_greater (core/NumericUtils.hpp:62-65) */
template<typename T>
__device__ __forceinline__ bool decidedly_greater(T a, T b) {
	return a > b && !almost_equal(a, b);
}

/* The losses that are a plain sum over the elements of a sample: the summand of _function ...
 *   LOSS_SQUARED                    loss/SquaredLoss.hpp:25-29             (o - y)^2
 *   LOSS_ABSOLUTE                   loss/AbsoluteLoss.hpp:25-30            |o - y|
 *   LOSS_BINARY_CROSS_ENTROPY       loss/BinaryCrossEntropyLoss.hpp:35-40  -(y ln(o + e) + (1 - y) ln((1 + e) - o))
 *   LOSS_CROSS_ENTROPY              loss/CrossEntropyLoss.hpp:33-38        -ln(o + e) y
 *   LOSS_KULLBACK_LEIBLER           loss/KullbackLeiblerLoss.hpp:32-39     -ln(o / (y + e) + e) y
 *   LOSS_MULTI_LABEL_HINGE          loss/MultiLabelHingeLoss.hpp:31-49     max(0, 1 - y o), squared in the SQUARED kind
 *   LOSS_MULTI_LABEL_LOG            loss/MultiLabelLogLoss.hpp:37-55       y ln(o + e) + (1 - y) ln(1 + e - o)
 * (the cross entropies are negated after the sum in the reference; negating each summand gives the same value) */
template<typename T, int KIND>
__device__ __forceinline__ T loss_summand(T o, T y, T eps) {
	const T one = (T) 1;
	if (KIND == LOSS_SQUARED) {
		const T d = o - y;
		return d * d;
	} else if (KIND == LOSS_ABSOLUTE) {
		return dev_abs(o - y);
	} else if (KIND == LOSS_BINARY_CROSS_ENTROPY) {
		return -(y * dev_log(o + eps) + (one - y) * dev_log((one + eps) - o));
	} else if (KIND == LOSS_CROSS_ENTROPY) {
		return -(dev_log(o + eps) * y);
	} else if (KIND == LOSS_KULLBACK_LEIBLER) {
		return -(dev_log(o / (y + eps) + eps) * y);
	} else if (KIND == LOSS_MULTI_LABEL_HINGE || KIND == LOSS_SQUARED_MULTI_LABEL_HINGE) {
		const T m = one - y * o;
		const T l = m > (T) 0 ? m : (T) 0;
		return KIND == LOSS_SQUARED_MULTI_LABEL_HINGE ? l * l : l;
	} else {
		return y * dev_log(o + eps) + (one - y) * dev_log(one + eps - o);
	}
}

/* ... and the element of _d_function:
 *   squared 2 (o - y) (SquaredLoss.hpp:30-33); absolute +1 for o - y >= 0, else -1 (AbsoluteLoss.hpp:31-35);
 *   binary cross entropy -(y / (o + e) - (1 - y) / ((1 + e) - o)) (BinaryCrossEntropyLoss.hpp:41-46);
 *   cross entropy and Kullback-Leibler -y / (o + e) (CrossEntropyLoss.hpp:39-42, KullbackLeiblerLoss.hpp:40-43);
 *   multi-label hinge -y, squared 2 o - 2 y, where 1 - y o is decidedly greater than 0, else 0
 *   (MultiLabelHingeLoss.hpp:50-71); multi-label log (y - o') / (o (1 - o)) with o' = o, or e where o is exactly 0
 *   (MultiLabelLogLoss.hpp:56-76). */
template<typename T, int KIND>
__device__ __forceinline__ T loss_derivative(T o, T y, T eps) {
	const T one = (T) 1;
	if (KIND == LOSS_SQUARED) {
		return (T) 2 * (o - y);
	} else if (KIND == LOSS_ABSOLUTE) {
		return o - y >= (T) 0 ? one : -one;
	} else if (KIND == LOSS_BINARY_CROSS_ENTROPY) {
		return -(y / (o + eps) - (one - y) / ((one + eps) - o));
	} else if (KIND == LOSS_CROSS_ENTROPY || KIND == LOSS_KULLBACK_LEIBLER) {
		return -y / (o + eps);
	} else if (KIND == LOSS_MULTI_LABEL_HINGE || KIND == LOSS_SQUARED_MULTI_LABEL_HINGE) {
		if (!decidedly_greater(one - y * o, (T) 0))
			return (T) 0;
		return KIND == LOSS_SQUARED_MULTI_LABEL_HINGE ? (T) 2 * o - (T) 2 * y : -y;
	} else {
		const T denominator = o * (one - o);
		const T numerator_o = o == (T) 0 ? o + eps : o;
		return (y - numerator_o) / denominator;
	}
}

/* L_n = sign * sum over the time steps and the elements of loss_summand. */
template<typename T, int KIND>
__global__ __launch_bounds__(ROWS * PARTS)
void summed_loss_kernel(int N, int T_steps, int V, T eps, T sign, const T* __restrict__ out, const T* __restrict__ obj,
		T* __restrict__ losses) {
	__shared__ T lds[ROWS * PARTS];
	const int n = blockIdx.x * ROWS + threadIdx.x;
	const bool live = n < N;
	const size_t cs = (size_t) N * T_steps;
	T total = (T) 0;
	for (int t = 0; t < T_steps; ++t) {              /* per-step losses add up (UniversalLoss.hpp:99-110) */
		T s = (T) 0;
		if (live) {
			const size_t base = (size_t) n + (size_t) N * t;
			for (int j = threadIdx.y; j < V; j += PARTS)
				s += loss_summand<T, KIND>(out[base + cs * j], obj[base + cs * j], eps);
		}
		total += row_combine<T, false>(s, lds);
	}
	if (live && threadIdx.y == 0)
		losses[n] = sign * total;
}

/* grad = scale * loss_derivative, element by element */
template<typename T, int KIND>
__global__ __launch_bounds__(256)
void loss_derivative_kernel(size_t total, T eps, T scale, const T* __restrict__ out, const T* __restrict__ obj,
		T* __restrict__ grad) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
		grad[i] = scale * loss_derivative<T, KIND>(out[i], obj[i], eps);
}

/* Hinge loss over one-hot objectives (loss/HingeLoss.hpp:31-99). The class c of a row is its last element that
 * almost equals 1; with s = out_c and m_j = out_j - s + 1 for j != c:
 *   GRAD = false: L_n = sign * sum_j max(0, m_j)  (squared: max(0, m_j)^2), summed over the time steps
 *   GRAD = true : grad_j = scale * g_j, g_j = 1 (squared: 2 m_j) where m_j is decidedly greater than 0, else 0,
 *                 and grad_c = -scale * sum_j g_j.
 * A row without a one (which the reference asserts against) gives NaN. */
template<typename T, bool SQUARED, bool GRAD>
__global__ __launch_bounds__(ROWS * PARTS)
void hinge_loss_kernel(int N, int T_steps, int V, T scale, const T* __restrict__ out, const T* __restrict__ obj,
		T* __restrict__ dst) {
	__shared__ T lds[ROWS * PARTS];
	const int n = blockIdx.x * ROWS + threadIdx.x;
	const bool live = n < N;
	const size_t cs = (size_t) N * T_steps;
	T total = (T) 0;
	for (int t = 0; t < T_steps; ++t) {
		const size_t base = (size_t) (live ? n : 0) + (size_t) N * t;
		T cls = (T) -1;
		if (live)
			for (int j = threadIdx.y; j < V; j += PARTS)
				if (almost_equal(obj[base + cs * j], (T) 1))
					cls = (T) j;
		const int c = (int) row_combine<T, true>(cls, lds);
		const T score = c >= 0 ? out[base + cs * c] : (T) NAN;
		T s = (T) 0;
		if (live)
			for (int j = threadIdx.y; j < V; j += PARTS) {
				if (j == c)
					continue;
				const T m = out[base + cs * j] - score + (T) 1;
				if (GRAD) {
					T g = (T) 0;
					if (decidedly_greater(m, (T) 0))
						g = SQUARED ? (T) 2 * m : (T) 1;
					else if (c < 0)
						g = (T) NAN;
					s += g;
					dst[base + cs * j] = scale * g;
				} else {
					const T l = m > (T) 0 ? m : (c < 0 ? (T) NAN : (T) 0);
					s += SQUARED ? l * l : l;
				}
			}
		s = row_combine<T, false>(s, lds);
		if (GRAD) {
			if (live && threadIdx.y == 0 && c >= 0)
				dst[base + cs * c] = scale * -s;
		} else
			total += s;
	}
	if (!GRAD && live && threadIdx.y == 0)
		dst[n] = scale * total;
}

/* Softmax cross entropy (loss/SoftmaxCrossEntropyLoss.hpp:33-50) with the reference's epsilon in
 * the softmax denominator: p_j = exp(o_j - max o) / (sum_i exp(o_i - max o) + eps).
 *   GRAD = false: L_n = - scale * sum_j log(p_j) * obj_j   (summed over time steps; scale is +1 or -1)
 *   GRAD = true : grad_j = scale * (p_j - obj_j) */
template<typename T, bool GRAD>
__global__ __launch_bounds__(ROWS * PARTS)
void softmax_ce_kernel(int N, int T_steps, int V, T eps, T scale, const T* __restrict__ out,
		const T* __restrict__ obj, T* __restrict__ dst) {
	__shared__ T lds[ROWS * PARTS];
	const int n = blockIdx.x * ROWS + threadIdx.x;
	const bool live = n < N;
	const size_t cs = (size_t) N * T_steps;
	T total = (T) 0;
	for (int t = 0; t < T_steps; ++t) {
		const size_t base = (size_t) (live ? n : 0) + (size_t) N * t;
		T mx = out[base];
		if (live)
			for (int j = threadIdx.y; j < V; j += PARTS) {
				const T e = out[base + cs * j];
				mx = e > mx ? e : mx;
			}
		mx = row_combine<T, true>(mx, lds);
		T s = (T) 0;
		if (live)
			for (int j = threadIdx.y; j < V; j += PARTS)
				s += dev_exp(out[base + cs * j] - mx);
		const T denom = row_combine<T, false>(s, lds) + eps;
		if (GRAD) {
			if (live)
				for (int j = threadIdx.y; j < V; j += PARTS) {
					const size_t i = base + cs * j;
					dst[i] = scale * (dev_exp(out[i] - mx) / denom - obj[i]);
				}
		} else {
			T l = (T) 0;
			if (live)
				for (int j = threadIdx.y; j < V; j += PARTS) {
					const size_t i = base + cs * j;
					l += dev_log(dev_exp(out[i] - mx) / denom) * obj[i];
				}
			total -= row_combine<T, false>(l, lds);
		}
	}
	if (!GRAD && live && threadIdx.y == 0)
		dst[n] = scale * total;
}

/* The _update_params bodies of the reference's optimizers, one element per thread, in place. The
 * scalars of a step (learning rate after annealing, bias corrections) come precomputed in `k`;
 * s0..s2 are the optimizer's per-parameter state matrices (zero after _fit).
 *   OPT_VANILLA_SGD   optimizer/VanillaSGDOptimizer.hpp:38-43        k: lr
 *   OPT_MOMENTUM_SGD  optimizer/MomentumSGDOptimizer.hpp:54-63       k: lr, momentum
 *   OPT_NESTEROV      optimizer/NesterovMomentumSGDOptimizer.hpp:43-55   k: lr, momentum
 *   OPT_ADAGRAD       optimizer/AdaGradOptimizer.hpp:50-70           k: lr, eps
 *   OPT_RMSPROP       optimizer/RMSPropOptimizer.hpp:43-47           k: lr, eps, l2_decay
 *   OPT_ADADELTA      optimizer/AdaDeltaOptimizer.hpp:53-67          k: decay, eps
 *   OPT_ADAM          optimizer/AdamOptimizer.hpp:66-82              k: d1, d2, lr * l1_corr, l2_corr, eps
 *   OPT_ADAMAX        optimizer/AdaMaxOptimizer.hpp:44-60            k: d1, d2, lr * l1_corr, -, eps
 *   OPT_NADAM         optimizer/NadamOptimizer.hpp:44-65             k: d1, d2, lr, l2_corr, eps, d1 * l1_corr, (1 - d1) * l1_next_corr
 *   OPT_AMSGRAD       optimizer/AMSGradOptimizer.hpp:48-66           k: d1, d2, lr, -, eps */
template<typename T, int RULE>
__device__ __forceinline__ T optimizer_element(const OptCoef<T>& k, T g, T v, T* __restrict__ s0, T* __restrict__ s1,
		T* __restrict__ s2, size_t i) {
	const T one = (T) 1;
	if (RULE == OPT_VANILLA_SGD) {
		return v - g * k.c[0];
	} else if (RULE == OPT_MOMENTUM_SGD) {
		const T s = s0[i] * k.c[1] + g * k.c[0];
		s0[i] = s;
		return v - s;
	} else if (RULE == OPT_NESTEROV) {
		const T old = s0[i];
		const T s = old * k.c[1] - g * k.c[0];
		s0[i] = s;
		return v + old * -k.c[1] + s * (one + k.c[1]);
	} else if (RULE == OPT_ADAGRAD || RULE == OPT_RMSPROP) {
		const T a = RULE == OPT_ADAGRAD ? s0[i] + g * g : s0[i] * (one - k.c[2]) + g * g * k.c[2];
		s0[i] = a;
		return v - g * k.c[0] / (dev_sqrt(a) + k.c[1]);
	} else if (RULE == OPT_ADADELTA) {
		const T a = s0[i] * (one - k.c[0]) + g * g * k.c[0];
		const T upd = -g * dev_sqrt(s1[i] + k.c[1]) / dev_sqrt(a + k.c[1]);
		s0[i] = a;
		s1[i] = s1[i] * (one - k.c[0]) + upd * upd * k.c[0];
		return v + upd;
	} else {
		const T m = s0[i] * (one - k.c[0]) + g * k.c[0];
		s0[i] = m;
		if (RULE == OPT_ADAMAX) {
			const T decayed = s1[i] * (one - k.c[1]), ag = g < (T) 0 ? -g : g;
			const T u = decayed > ag ? decayed : ag;
			s1[i] = u;
			return v - (m * k.c[2]) / (u + k.c[4]);
		}
		const T sq = s1[i] * (one - k.c[1]) + g * g * k.c[1];
		s1[i] = sq;
		if (RULE == OPT_ADAM)
			return v - (m * k.c[2]) / dev_sqrt(sq * k.c[3] + k.c[4]);
		if (RULE == OPT_NADAM)
			return v - ((g * k.c[5] + m * k.c[6]) * k.c[2]) / dev_sqrt(sq * k.c[3] + k.c[4]);
		/* OPT_AMSGRAD */
		const T prev = s2[i];
		const T mx = sq > prev ? sq : prev;
		s2[i] = mx;
		return v - (m * k.c[2]) / dev_sqrt(mx + k.c[4]);
	}
}

/* Parameters::regularize before the update (optimizer/SGDOptimizer.hpp:59-63, parameters/StandardParameters.hpp:133-136):
 * the gradient plus d_function of the parameter's regularization at its values - L1 (e >= 0 ? lambda : -lambda,
 * parameter_regularization/L1ParameterRegularization.hpp:35-37), L2 (e * lambda, L2ParameterRegularization.hpp:35-37)
 * or both (ElasticNetParameterRegularization.hpp:40-42). Both lambdas zero: no regularization, the gradient as it is. */
template<typename T>
__device__ __forceinline__ T regularized_gradient(T g, T v, T l1, T l2) {
	if (l1 == (T) 0 && l2 == (T) 0)
		return g;
	const T sign_term = v >= (T) 0 ? l1 : -l1;
	const T reg = l2 == (T) 0 ? sign_term : (l1 == (T) 0 ? v * l2 : sign_term + v * l2);
	return g + reg;
}

template<typename T, int RULE>
__global__ __launch_bounds__(256)
void optimizer_update_kernel(size_t total, OptCoef<T> k, T* __restrict__ grad, T* __restrict__ s0, T* __restrict__ s1,
		T* __restrict__ s2, T* __restrict__ values, bool reset_grad, T l1, T l2) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		values[i] = optimizer_element<T, RULE>(k, regularized_gradient(grad[i], values[i], l1, l2), values[i], s0, s1, s2, i);
		if (reset_grad)                 /* Parameters::reset_grad after the update (optimizer/SGDOptimizer.hpp:68-70) */
			grad[i] = (T) 0;
	}
}

template<typename T>
__global__ __launch_bounds__(256)
void regularization_sums_kernel(size_t n, const T* __restrict__ values, T* __restrict__ sums) {
	__shared__ T part[2][256];
	T a = (T) 0, q = (T) 0;
	for (size_t i = threadIdx.x; i < n; i += 256) {
		const T v = values[i];
		a += v < (T) 0 ? -v : v;
		q += v * v;
	}
	part[0][threadIdx.x] = a;
	part[1][threadIdx.x] = q;
	__syncthreads();
	for (int w = 128; w > 0; w >>= 1) {
		if ((int) threadIdx.x < w) {
			part[0][threadIdx.x] += part[0][threadIdx.x + w];
			part[1][threadIdx.x] += part[1][threadIdx.x + w];
		}
		__syncthreads();
	}
	if (threadIdx.x == 0) {
		sums[0] = part[0][0];
		sums[1] = part[1][0];
	}
}

/* The constraints of a Parameters object on its values or on its gradient (parameters/StandardParameters.hpp:150-182),
 * in the order set_values and accumulate_grad enforce them (:109-111, :120-122): clip to [-clip, clip], then scale by
 * max_l1 / norm() where the norm() - the Euclidean norm: that is what the "L1" constraint calls - exceeds max_l1, then
 * scale by max_l2 / squaredNorm() where the squared norm (what the "L2" constraint compares with its limit) exceeds
 * max_l2. A limit that is not decidedly greater than zero is off. One block: the sums are taken thread by thread in a
 * fixed order, then by a fixed tree, so the result is reproducible. */
template<typename T>
__device__ __forceinline__ T block_sum_of_squares(size_t n, const T* m, T (&part)[256]) {
	T q = (T) 0;
	for (size_t i = threadIdx.x; i < n; i += 256)
		q += m[i] * m[i];
	part[threadIdx.x] = q;
	__syncthreads();
	for (int w = 128; w > 0; w >>= 1) {
		if ((int) threadIdx.x < w)
			part[threadIdx.x] += part[threadIdx.x + w];
		__syncthreads();
	}
	const T total = part[0];
	__syncthreads();
	return total;
}

template<typename T>
__global__ __launch_bounds__(256)
void constrain_kernel(size_t n, T* __restrict__ m, T clip, T max_l1, T max_l2) {
	__shared__ T part[256];
	if (clip > (T) 0) {
		for (size_t i = threadIdx.x; i < n; i += 256) {
			const T v = m[i];
			m[i] = v > clip ? clip : (v < -clip ? -clip : v);
		}
		__syncthreads();
	}
	if (max_l1 > (T) 0) {
		const T norm = dev_sqrt(block_sum_of_squares<T>(n, m, part));
		if (norm > max_l1) {
			const T scale = max_l1 / norm;
			for (size_t i = threadIdx.x; i < n; i += 256)
				m[i] *= scale;
		}
		__syncthreads();
	}
	if (max_l2 > (T) 0) {
		const T sq = block_sum_of_squares<T>(n, m, part);
		if (sq > max_l2) {
			const T scale = max_l2 / sq;
			for (size_t i = threadIdx.x; i < n; i += 256)
				m[i] *= scale;
		}
	}
}

/* grad += d_function of the regularization at the values: Parameters::regularize as a step of its own, for parameters
 * whose gradient is constrained (the constraints apply to the sum, StandardParameters.hpp:133-136 through :114-123). */
template<typename T>
__global__ __launch_bounds__(256)
void add_regularization_kernel(size_t n, const T* __restrict__ values, T* __restrict__ grad, T l1, T l2) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
		grad[i] = regularized_gradient(grad[i], values[i], l1, l2);
}

/* The update and gradient reset of up to OPT_BATCH parameters in one launch (blockIdx.y picks the parameter,
 * blockIdx.x a run of 1024 elements, or a 32 x 32 tile of the matrix). A convolution or dense weight matrix may
 * bring its prepared layouts along (the forward layout wt[k][f] and the input-gradient layout wd[tap + RHW * f][c],
 * both zero-padded when they were first built): the new values are written there as well, which saves the two
 * re-layout launches of the next pass. The matrix is column-major (k fastest) and wt is f fastest, so a tile goes
 * through LDS and both sides are accessed along their contiguous index. */
/* the gradient of element i: what has been accumulated plus the partial sums that still wait, these added up first, in
 * ascending order from zero (the order and grouping of reduce_partials_many for so few of them) */
template<typename T>
__device__ __forceinline__ T whole_gradient(const OptParam<T>& q, size_t i) {
	T g = q.grad[i];
	if (q.parts != nullptr) {
		T t = (T) 0;
		for (int s = 0; s < q.splits; ++s)
			t += q.parts[(size_t) s * q.n + i];
		g += t;
	}
	return g;
}

template<typename T, int RULE>
__global__ __launch_bounds__(256)
void optimizer_step_many_kernel(OptBatch<T> batch, OptCoef<T> k) {
	__shared__ T tile[32][33];
	const OptParam<T>& q = batch.p[blockIdx.y];
	const int tid = threadIdx.x;
	if (!q.wt_fwd && !q.wt_dgrad) {
		#pragma unroll
		for (int j = 0; j < 4; ++j) {
			const size_t i = (size_t) blockIdx.x * 1024 + tid + 256 * j;
			if (i < q.n) {
				q.values[i] = optimizer_element<T, RULE>(k, regularized_gradient(whole_gradient(q, i), q.values[i], q.l1, q.l2), q.values[i], q.s0, q.s1,
						q.s2, i);
				q.grad[i] = (T) 0;
			}
		}
		return;
	}
	const int F = (int) (q.n / (size_t) q.K);
	const int tiles_k = (q.K + 31) / 32;
	if ((int) blockIdx.x >= tiles_k * ((F + 31) / 32))
		return;
	const int k0 = ((int) blockIdx.x % tiles_k) * 32, f0 = ((int) blockIdx.x / tiles_k) * 32;
	const int a = tid % 32, b = tid / 32;
	#pragma unroll
	for (int j = 0; j < 4; ++j) {
		const int row = k0 + a, f = f0 + b + 8 * j;
		if (row < q.K && f < F) {
			const size_t i = (size_t) row + (size_t) q.K * f;
			const T v = optimizer_element<T, RULE>(k, regularized_gradient(whole_gradient(q, i), q.values[i], q.l1, q.l2), q.values[i], q.s0, q.s1,
					q.s2, i);
			q.values[i] = v;
			q.grad[i] = (T) 0;
			tile[b + 8 * j][a] = v;
			if (q.wt_dgrad) {
				const unsigned tap = (unsigned) row % (unsigned) q.RHW, c = (unsigned) row / (unsigned) q.RHW;
				q.wt_dgrad[(size_t) (tap + (unsigned) q.RHW * f) * q.ldw_dgrad + c] = v;
			}
		}
	}
	if (!q.wt_fwd)
		return;
	__syncthreads();
	#pragma unroll
	for (int j = 0; j < 4; ++j) {
		const int row = k0 + b + 8 * j, f = f0 + a;
		if (row < q.K && f < F)
			q.wt_fwd[(size_t) row * q.ldw_fwd + f] = tile[a][b + 8 * j];
	}
}

unsigned flat_grid(size_t work_items) {
	const size_t blocks = (work_items + 255) / 256;
	return (unsigned) std::max<size_t>(1, std::min<size_t>(blocks, 256 * 16));
}

void check_launch() {
	CATTLE_HIP_CHECK(hipGetLastError());
}

} /* namespace */

/* kind | LOSS_NEGATED is the loss wrapped in NegatedLoss (loss/NegatedLoss.hpp:41-46): both results change sign. */
template<typename T>
void loss_function(int kind, int N, int T_steps, int V, T eps, const T* out, const T* obj, T* losses) {
	if (N == 0)
		return;
	const T sign = (kind & LOSS_NEGATED) ? (T) -1 : (T) 1;
	kind &= ~LOSS_NEGATED;
	const dim3 block(ROWS, PARTS);
	const unsigned grid = (unsigned) ((N + ROWS - 1) / ROWS);
#define CATTLE_HIP_SUMMED_LOSS(KIND) \
	case KIND: \
		summed_loss_kernel<T, KIND><<<grid, block, 0, stream()>>>(N, T_steps, V, eps, sign, out, obj, losses); \
		break;
	switch (kind) {
	CATTLE_HIP_SUMMED_LOSS(LOSS_SQUARED)
	CATTLE_HIP_SUMMED_LOSS(LOSS_ABSOLUTE)
	CATTLE_HIP_SUMMED_LOSS(LOSS_CROSS_ENTROPY)
	CATTLE_HIP_SUMMED_LOSS(LOSS_KULLBACK_LEIBLER)
	CATTLE_HIP_SUMMED_LOSS(LOSS_MULTI_LABEL_HINGE)
	CATTLE_HIP_SUMMED_LOSS(LOSS_SQUARED_MULTI_LABEL_HINGE)
	CATTLE_HIP_SUMMED_LOSS(LOSS_MULTI_LABEL_LOG)
	case LOSS_BINARY_CROSS_ENTROPY:
		if (V != 1)
			throw Error(ERR_INVALID, "the binary cross entropy loss takes one value per sample and time step");
		summed_loss_kernel<T, LOSS_BINARY_CROSS_ENTROPY><<<grid, block, 0, stream()>>>(N, T_steps, V, eps, sign, out, obj, losses);
		break;
	case LOSS_SOFTMAX_CROSS_ENTROPY:
		softmax_ce_kernel<T, false><<<grid, block, 0, stream()>>>(N, T_steps, V, eps, sign, out, obj, losses);
		break;
	case LOSS_HINGE:
		hinge_loss_kernel<T, false, false><<<grid, block, 0, stream()>>>(N, T_steps, V, sign, out, obj, losses);
		break;
	case LOSS_SQUARED_HINGE:
		hinge_loss_kernel<T, true, false><<<grid, block, 0, stream()>>>(N, T_steps, V, sign, out, obj, losses);
		break;
	default:
		throw Error(ERR_INVALID, "unknown loss kind");
	}
#undef CATTLE_HIP_SUMMED_LOSS
	check_launch();
}

template<typename T>
void loss_d_function(int kind, int N, int T_steps, int V, T eps, T scale, const T* out, const T* obj, T* grad) {
	const size_t total = (size_t) N * T_steps * V;
	if (total == 0)
		return;
	if (kind & LOSS_NEGATED)
		scale = -scale;
	kind &= ~LOSS_NEGATED;
	const dim3 block(ROWS, PARTS);
	const unsigned rows_grid = (unsigned) ((N + ROWS - 1) / ROWS);
#define CATTLE_HIP_LOSS_DERIVATIVE(KIND) \
	case KIND: \
		loss_derivative_kernel<T, KIND><<<flat_grid(total), 256, 0, stream()>>>(total, eps, scale, out, obj, grad); \
		break;
	switch (kind) {
	CATTLE_HIP_LOSS_DERIVATIVE(LOSS_SQUARED)
	CATTLE_HIP_LOSS_DERIVATIVE(LOSS_ABSOLUTE)
	CATTLE_HIP_LOSS_DERIVATIVE(LOSS_CROSS_ENTROPY)
	CATTLE_HIP_LOSS_DERIVATIVE(LOSS_KULLBACK_LEIBLER)
	CATTLE_HIP_LOSS_DERIVATIVE(LOSS_MULTI_LABEL_HINGE)
	CATTLE_HIP_LOSS_DERIVATIVE(LOSS_SQUARED_MULTI_LABEL_HINGE)
	CATTLE_HIP_LOSS_DERIVATIVE(LOSS_MULTI_LABEL_LOG)
	case LOSS_BINARY_CROSS_ENTROPY:
		if (V != 1)
			throw Error(ERR_INVALID, "the binary cross entropy loss takes one value per sample and time step");
		loss_derivative_kernel<T, LOSS_BINARY_CROSS_ENTROPY><<<flat_grid(total), 256, 0, stream()>>>(total, eps, scale, out, obj, grad);
		break;
	case LOSS_SOFTMAX_CROSS_ENTROPY:
		softmax_ce_kernel<T, true><<<rows_grid, block, 0, stream()>>>(N, T_steps, V, eps, scale, out, obj, grad);
		break;
	case LOSS_HINGE:
		hinge_loss_kernel<T, false, true><<<rows_grid, block, 0, stream()>>>(N, T_steps, V, scale, out, obj, grad);
		break;
	case LOSS_SQUARED_HINGE:
		hinge_loss_kernel<T, true, true><<<rows_grid, block, 0, stream()>>>(N, T_steps, V, scale, out, obj, grad);
		break;
	default:
		throw Error(ERR_INVALID, "unknown loss kind");
	}
#undef CATTLE_HIP_LOSS_DERIVATIVE
	check_launch();
}

int optimizer_state_count(int rule) {
	switch (rule) {
	case OPT_VANILLA_SGD: return 0;
	case OPT_MOMENTUM_SGD: case OPT_NESTEROV: case OPT_ADAGRAD: case OPT_RMSPROP: return 1;
	case OPT_ADADELTA: case OPT_ADAM: case OPT_ADAMAX: case OPT_NADAM: return 2;
	case OPT_AMSGRAD: return 3;
	default: throw Error(ERR_INVALID, "unknown optimizer");
	}
}

/* The scalars of one optimizer step. */
template<typename T>
OptCoef<T> optimizer_coefficients(int rule, const double hyper[4], size_t epoch, size_t timestep) {
	OptCoef<T> k;
	for (int i = 0; i < 8; ++i)
		k.c[i] = (T) 0;
	const T h0 = (T) hyper[0], h1 = (T) hyper[1], h2 = (T) hyper[2], h3 = (T) hyper[3];
	const T one = (T) 1;
	/* every scalar of the step is formed in T, as the reference forms it in Scalar */
	switch (rule) {
	case OPT_VANILLA_SGD:                /* hyper: learning_rate */
		CATTLE_HIP_REQUIRE(h0 > 0, "learning rate must be positive");
		k.c[0] = h0;
		break;
	case OPT_MOMENTUM_SGD: case OPT_NESTEROV:     /* hyper: init_learning_rate, annealing_rate, momentum */
		CATTLE_HIP_REQUIRE(h0 > 0 && h1 >= 0 && h2 > 0 && h2 < 1, "momentum SGD: learning rate > 0, annealing rate >= 0, 0 < momentum < 1");
		k.c[0] = h0 / (one + h1 * (T) epoch);       /* calculate_learning_rate (MomentumSGDOptimizer.hpp:70-72) */
		k.c[1] = h2;
		break;
	case OPT_ADAGRAD:                    /* hyper: learning_rate, epsilon */
		CATTLE_HIP_REQUIRE(h0 > 0 && h1 > 0, "AdaGrad: learning rate and epsilon must be positive");
		k.c[0] = h0; k.c[1] = h1;
		break;
	case OPT_RMSPROP:                    /* hyper: learning_rate, l2_decay, epsilon */
		CATTLE_HIP_REQUIRE(h0 > 0 && h1 >= 0 && h1 <= 1 && h2 > 0, "RMSProp: learning rate, epsilon > 0, decay in [0,1]");
		k.c[0] = h0; k.c[1] = h2; k.c[2] = h1;
		break;
	case OPT_ADADELTA:                   /* hyper: decay, epsilon */
		CATTLE_HIP_REQUIRE(h0 >= 0 && h0 <= 1 && h1 > 0, "AdaDelta: decay in [0,1], epsilon > 0");
		k.c[0] = h0; k.c[1] = h1;
		break;
	case OPT_ADAM: case OPT_ADAMAX: case OPT_NADAM: case OPT_AMSGRAD: {      /* hyper: learning_rate, l1_decay, l2_decay, epsilon */
		CATTLE_HIP_REQUIRE(h0 > 0, "learning rate must be positive");
		CATTLE_HIP_REQUIRE(h1 >= 0 && h1 <= 1 && h2 >= 0 && h2 <= 1, "decay rates must lie in [0,1]");
		CATTLE_HIP_REQUIRE(h3 > 0, "epsilon must be positive");
		const T l1_corr = one / (one - (T) std::pow(one - h1, (T) (timestep + 1)) + h3);
		const T l1_next_corr = one / (one - (T) std::pow(one - h1, (T) (timestep + 2)) + h3);
		const T l2_corr = one / (one - (T) std::pow(one - h2, (T) (timestep + 1)) + h3);
		k.c[0] = h1; k.c[1] = h2; k.c[3] = l2_corr; k.c[4] = h3;
		k.c[2] = rule == OPT_ADAM || rule == OPT_ADAMAX ? h0 * l1_corr : h0;
		k.c[5] = h1 * l1_corr;
		k.c[6] = (one - h1) * l1_next_corr;
		break;
	}
	default:
		throw Error(ERR_INVALID, "unknown optimizer");
	}
	return k;
}

#define CATTLE_HIP_OPT_DISPATCH(rule, LAUNCH) \
	switch (rule) { \
	case OPT_VANILLA_SGD: LAUNCH(OPT_VANILLA_SGD); break; \
	case OPT_MOMENTUM_SGD: LAUNCH(OPT_MOMENTUM_SGD); break; \
	case OPT_NESTEROV: LAUNCH(OPT_NESTEROV); break; \
	case OPT_ADAGRAD: LAUNCH(OPT_ADAGRAD); break; \
	case OPT_RMSPROP: LAUNCH(OPT_RMSPROP); break; \
	case OPT_ADADELTA: LAUNCH(OPT_ADADELTA); break; \
	case OPT_ADAM: LAUNCH(OPT_ADAM); break; \
	case OPT_ADAMAX: LAUNCH(OPT_ADAMAX); break; \
	case OPT_NADAM: LAUNCH(OPT_NADAM); break; \
	default: LAUNCH(OPT_AMSGRAD); break; \
	}

/* sums[0] = sum |v|, sums[1] = sum v^2: what the regularization penalties are made of (L1: lambda * sum |v|,
 * L2: 0.5 * lambda * sum v^2; parameter_regularization/L1ParameterRegularization.hpp:32-34,
 * L2ParameterRegularization.hpp:32-34). One block, fixed order: parameters are at most a few million values. */
template<typename T>
void regularization_sums(size_t n, const T* values, T* sums) {
	regularization_sums_kernel<T><<<1, 256, 0, stream()>>>(n, values, sums);
	check_launch();
}

/* NumericUtils::decidedly_greater(limit, 0) with its default epsilons (core/NumericUtils.hpp:42-65) */
template<typename T>
T active_limit(double limit) {
	const T l = (T) limit;
	return l > std::numeric_limits<T>::epsilon() ? l : (T) 0;
}

template<typename T>
void constrain_matrix(size_t n, T* m, double clip, double max_l1, double max_l2) {
	const T c = active_limit<T>(clip), a = active_limit<T>(max_l1), b = active_limit<T>(max_l2);
	if (n == 0 || (c == (T) 0 && a == (T) 0 && b == (T) 0))
		return;
	constrain_kernel<T><<<1, 256, 0, stream()>>>(n, m, c, a, b);
	check_launch();
}

template<typename T>
void add_regularization(size_t n, const T* values, T* grad, T l1, T l2) {
	if (n == 0 || (l1 == (T) 0 && l2 == (T) 0))
		return;
	add_regularization_kernel<T><<<flat_grid(n), 256, 0, stream()>>>(n, values, grad, l1, l2);
	check_launch();
}

template<typename T>
void optimizer_update(int rule, const double hyper[4], size_t epoch, size_t timestep, size_t n, T* grad, T* s0, T* s1,
		T* s2, T* values, bool reset_grad, T l1, T l2) {
	if (n == 0)
		return;
	const OptCoef<T> k = optimizer_coefficients<T>(rule, hyper, epoch, timestep);
	const unsigned grid = flat_grid(n);
#define CATTLE_HIP_LAUNCH_ONE(R) optimizer_update_kernel<T, R><<<grid, 256, 0, stream()>>>(n, k, grad, s0, s1, s2, values, reset_grad, l1, l2)
	CATTLE_HIP_OPT_DISPATCH(rule, CATTLE_HIP_LAUNCH_ONE)
#undef CATTLE_HIP_LAUNCH_ONE
	check_launch();
}

template<typename T>
void optimizer_step_many(int rule, const double hyper[4], size_t epoch, size_t timestep, const OptBatch<T>& batch) {
	if (batch.count == 0)
		return;
	CATTLE_HIP_REQUIRE(batch.count <= OPT_BATCH, "too many parameters in one optimizer launch");
	const OptCoef<T> k = optimizer_coefficients<T>(rule, hyper, epoch, timestep);
	size_t blocks = 1;        /* of the parameter that needs the most: runs of 1024 elements or 32 x 32 tiles */
	for (int i = 0; i < batch.count; ++i) {
		const OptParam<T>& q = batch.p[i];
		if (q.wt_fwd || q.wt_dgrad)
			blocks = std::max(blocks, (size_t) ((q.K + 31) / 32) * ((q.n / (size_t) q.K + 31) / 32));
		else
			blocks = std::max(blocks, (q.n + 1023) / 1024);
	}
	CATTLE_HIP_REQUIRE(blocks <= 2147483647u, "parameter too large for one optimizer launch");
	const dim3 grid((unsigned) blocks, (unsigned) batch.count);
#define CATTLE_HIP_LAUNCH_MANY(R) optimizer_step_many_kernel<T, R><<<grid, 256, 0, stream()>>>(batch, k)
	CATTLE_HIP_OPT_DISPATCH(rule, CATTLE_HIP_LAUNCH_MANY)
#undef CATTLE_HIP_LAUNCH_MANY
	check_launch();
}

#define CATTLE_HIP_INSTANTIATE_TRAIN(T) \
template void loss_function<T>(int, int, int, int, T, const T*, const T*, T*); \
template void loss_d_function<T>(int, int, int, int, T, T, const T*, const T*, T*); \
template void optimizer_update<T>(int, const double*, size_t, size_t, size_t, T*, T*, T*, T*, T*, bool, T, T); \
template void regularization_sums<T>(size_t, const T*, T*); \
template void constrain_matrix<T>(size_t, T*, double, double, double); \
template void add_regularization<T>(size_t, const T*, T*, T, T); \
template void optimizer_step_many<T>(int, const double*, size_t, size_t, const OptBatch<T>&);

CATTLE_HIP_INSTANTIATE_TRAIN(float)
CATTLE_HIP_INSTANTIATE_TRAIN(double)

} /* namespace cattle_hip */
