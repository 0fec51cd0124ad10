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

/* Squared error (loss/SquaredLoss.hpp:25-34): L_n = sum_j (out - obj)^2. */
template<typename T>
__global__ __launch_bounds__(ROWS * PARTS)
void squared_loss_kernel(int N, int T_steps, int V, const T* __restrict__ out, const T* __restrict__ obj,
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
			for (int j = threadIdx.y; j < V; j += PARTS) {
				const T d = out[base + cs * j] - obj[base + cs * j];
				s += d * d;
			}
		}
		total += row_combine<T, false>(s, lds);
	}
	if (live && threadIdx.y == 0)
		losses[n] = total;
}

/* grad = scale * 2 (out - obj) */
template<typename T>
__global__ __launch_bounds__(256)
void squared_loss_grad_kernel(size_t total, T two_scale, const T* __restrict__ out, const T* __restrict__ obj,
		T* __restrict__ grad) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
		grad[i] = two_scale * (out[i] - obj[i]);
}

/* Softmax cross entropy (loss/SoftmaxCrossEntropyLoss.hpp:33-50) with the reference's epsilon in
 * the softmax denominator: p_j = exp(o_j - max o) / (sum_i exp(o_i - max o) + eps).
 *   GRAD = false: L_n = - sum_j log(p_j) * obj_j   (summed over time steps)
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
		dst[n] = total;
}

/* values -= grad * lr  (optimizer/VanillaSGDOptimizer.hpp:38-43) */
template<typename T>
__global__ __launch_bounds__(256)
void sgd_update_kernel(size_t total, T lr, const T* __restrict__ grad, T* __restrict__ values) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
		values[i] -= grad[i] * lr;
}

/* optimizer/AdamOptimizer.hpp:66-82:
 *   m = m (1 - d1) + g d1;  v = v (1 - d2) + g g d2;
 *   values -= (m * (lr * l1_corr)) / sqrt(v * l2_corr + eps)      (epsilon inside the root) */
template<typename T>
__global__ __launch_bounds__(256)
void adam_update_kernel(size_t total, T d1, T d2, T lr_corr, T l2_corr, T eps, const T* __restrict__ grad,
		T* __restrict__ m, T* __restrict__ v, T* __restrict__ values) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		const T g = grad[i];
		const T mi = m[i] * ((T) 1 - d1) + g * d1;
		const T vi = v[i] * ((T) 1 - d2) + g * g * d2;
		m[i] = mi;
		v[i] = vi;
		values[i] -= (mi * lr_corr) / dev_sqrt(vi * l2_corr + eps);
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

template<typename T>
void loss_function(int kind, int N, int T_steps, int V, T eps, const T* out, const T* obj, T* losses) {
	if (N == 0)
		return;
	const dim3 block(ROWS, PARTS);
	const unsigned grid = (unsigned) ((N + ROWS - 1) / ROWS);
	switch (kind) {
	case LOSS_SQUARED:
		squared_loss_kernel<T><<<grid, block, 0, stream()>>>(N, T_steps, V, out, obj, losses);
		break;
	case LOSS_SOFTMAX_CROSS_ENTROPY:
		softmax_ce_kernel<T, false><<<grid, block, 0, stream()>>>(N, T_steps, V, eps, (T) 1, out, obj, losses);
		break;
	default:
		throw Error(ERR_INVALID, "unknown loss kind");
	}
	check_launch();
}

template<typename T>
void loss_d_function(int kind, int N, int T_steps, int V, T eps, T scale, const T* out, const T* obj, T* grad) {
	const size_t total = (size_t) N * T_steps * V;
	if (total == 0)
		return;
	switch (kind) {
	case LOSS_SQUARED:
		squared_loss_grad_kernel<T><<<flat_grid(total), 256, 0, stream()>>>(total, (T) 2 * scale, out, obj, grad);
		break;
	case LOSS_SOFTMAX_CROSS_ENTROPY:
		softmax_ce_kernel<T, true><<<(unsigned) ((N + ROWS - 1) / ROWS), dim3(ROWS, PARTS), 0, stream()>>>(
				N, T_steps, V, eps, scale, out, obj, grad);
		break;
	default:
		throw Error(ERR_INVALID, "unknown loss kind");
	}
	check_launch();
}

template<typename T>
void sgd_update(size_t n, T lr, const T* grad, T* values) {
	if (n == 0)
		return;
	sgd_update_kernel<T><<<flat_grid(n), 256, 0, stream()>>>(n, lr, grad, values);
	check_launch();
}

template<typename T>
void adam_update(size_t n, T lr, T l1_decay, T l2_decay, T eps, size_t timestep, const T* grad, T* m, T* v,
		T* values) {
	if (n == 0)
		return;
	/* the bias corrections are scalars of the step, computed in T as the reference does (:67-68) */
	const T l1_corr = (T) 1 / ((T) 1 - (T) std::pow((T) 1 - l1_decay, (T) (timestep + 1)) + eps);
	const T l2_corr = (T) 1 / ((T) 1 - (T) std::pow((T) 1 - l2_decay, (T) (timestep + 1)) + eps);
	adam_update_kernel<T><<<flat_grid(n), 256, 0, stream()>>>(n, l1_decay, l2_decay, lr * l1_corr, l2_corr, eps,
			grad, m, v, values);
	check_launch();
}

#define CATTLE_HIP_INSTANTIATE_TRAIN(T) \
template void loss_function<T>(int, int, int, int, T, const T*, const T*, T*); \
template void loss_d_function<T>(int, int, int, int, T, T, const T*, const T*, T*); \
template void sgd_update<T>(size_t, T, const T*, T*); \
template void adam_update<T>(size_t, T, T, T, T, size_t, const T*, T*, T*, T*);

CATTLE_HIP_INSTANTIATE_TRAIN(float)
CATTLE_HIP_INSTANTIATE_TRAIN(double)

} /* namespace cattle_hip */
