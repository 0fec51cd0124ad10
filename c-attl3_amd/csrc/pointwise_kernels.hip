/*
 * pointwise_kernels.hip — HBM-bound kernels: activations, softmax, batch norm, pooling (gfx950).
 *
 * Every tensor is the reference's column-major (N,H,W,C) buffer. Consecutive threads always walk
 * the contiguous N (then H) direction, element-wise kernels use 16-byte accesses, and every
 * reduction is a fixed-order two-stage sum (wavefront shuffles + LDS, then partials in ascending
 * order), so results are reproducible run to run; no atomics are used anywhere.
 */
#include "common.hpp"
#include "act_math.hpp"
#include "lstm_math.hpp"

#include <algorithm>
#include <limits>
#include <type_traits>

namespace cattle_hip {

namespace {

template<typename T> struct Pack { static constexpr int V = 16 / (int) sizeof(T); typedef T type __attribute__((ext_vector_type(16 / sizeof(T)))); };

template<typename T, int KIND, bool VECTOR>
__global__ __launch_bounds__(256)
void act_forward_kernel(size_t n, T p, const T* __restrict__ x, T* __restrict__ y) {
	constexpr int V = VECTOR ? Pack<T>::V : 1;
	typedef typename Pack<T>::type vt;
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	const size_t nv = n / V;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
		if constexpr (VECTOR) {
			vt a = __builtin_nontemporal_load(reinterpret_cast<const vt*>(x) + i), o;
			#pragma unroll
			for (int e = 0; e < V; ++e)
				o[e] = act_f<T, KIND>(a[e], p);
			__builtin_nontemporal_store(o, reinterpret_cast<vt*>(y) + i);
		} else {
			y[i] = act_f<T, KIND>(x[i], p);
		}
	}
	if (VECTOR && blockIdx.x == 0 && threadIdx.x < n - nv * V) {
		const size_t i = nv * V + threadIdx.x;
		y[i] = act_f<T, KIND>(x[i], p);
	}
}

template<typename T, int KIND, bool VECTOR>
__global__ __launch_bounds__(256)
void act_backward_kernel(size_t n, T p, const T* __restrict__ x, const T* __restrict__ y, const T* __restrict__ g,
		T* __restrict__ dx) {
	constexpr int V = VECTOR ? Pack<T>::V : 1;
	typedef typename Pack<T>::type vt;
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	const size_t nv = n / V;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
		if constexpr (VECTOR) {
			vt xv = {0}, yv = {0}, o;
			if (act_needs_x(KIND))
				xv = __builtin_nontemporal_load(reinterpret_cast<const vt*>(x) + i);
			if (act_needs_y(KIND))
				yv = __builtin_nontemporal_load(reinterpret_cast<const vt*>(y) + i);
			const vt gv = __builtin_nontemporal_load(reinterpret_cast<const vt*>(g) + i);
			#pragma unroll
			for (int e = 0; e < V; ++e)
				o[e] = act_b<T, KIND>(xv[e], yv[e], gv[e], p);
			__builtin_nontemporal_store(o, reinterpret_cast<vt*>(dx) + i);
		} else {
			dx[i] = act_b<T, KIND>(act_needs_x(KIND) ? x[i] : (T) 0, act_needs_y(KIND) ? y[i] : (T) 0, g[i], p);
		}
	}
	if (VECTOR && blockIdx.x == 0 && threadIdx.x < n - nv * V) {
		const size_t i = nv * V + threadIdx.x;
		dx[i] = act_b<T, KIND>(act_needs_x(KIND) ? x[i] : (T) 0, act_needs_y(KIND) ? y[i] : (T) 0, g[i], p);
	}
}

bool aligned16(const void* p) {
	return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

unsigned stream_grid(size_t work_items) {
	const size_t blocks = (work_items + 255) / 256;
	return (unsigned) std::max<size_t>(1, std::min<size_t>(blocks, (size_t) 1 << 22));
}

template<typename T, int KIND>
void act_forward_kind(size_t n, T p, const T* x, T* y) {
	if (aligned16(x) && aligned16(y))
		act_forward_kernel<T, KIND, true><<<stream_grid(n / Pack<T>::V), 256, 0, stream()>>>(n, p, x, y);
	else
		act_forward_kernel<T, KIND, false><<<stream_grid(n), 256, 0, stream()>>>(n, p, x, y);
}

template<typename T, int KIND>
void act_backward_kind(size_t n, T p, const T* x, const T* y, const T* g, T* dx) {
	CATTLE_HIP_REQUIRE(!act_needs_x(KIND) || x, "activation backward needs the cached input");
	CATTLE_HIP_REQUIRE(!act_needs_y(KIND) || y, "activation backward needs the cached output");
	const bool al = aligned16(g) && aligned16(dx) && (!act_needs_x(KIND) || aligned16(x)) && (!act_needs_y(KIND) || aligned16(y));
	if (al)
		act_backward_kernel<T, KIND, true><<<stream_grid(n / Pack<T>::V), 256, 0, stream()>>>(n, p, x, y, g, dx);
	else
		act_backward_kernel<T, KIND, false><<<stream_grid(n), 256, 0, stream()>>>(n, p, x, y, g, dx);
}

/* Sum over the 64 lanes of a wavefront; the result is valid in lane 0. */
template<typename T>
__device__ __forceinline__ T wave_sum(T v) {
	#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		v += __shfl_down(v, off, 64);
	return v;
}

/* Sum over a 256-thread block (4 wavefronts); the result is returned to every thread. */
template<typename T>
__device__ __forceinline__ T block_sum_256(T v, T* lds) {
	v = wave_sum(v);
	__syncthreads();
	if (threadIdx.x % 64 == 0)
		lds[threadIdx.x / 64] = v;
	__syncthreads();
	return ((lds[0] + lds[1]) + lds[2]) + lds[3];
}

/* ----------------------------------------------------------------------------------------------
 * Softmax over the columns of an N x V column-major matrix, one thread per row
 * (layer/activation/SoftmaxActivationLayer.hpp:49-78).
 * -------------------------------------------------------------------------------------------- */
template<typename T>
__global__ void softmax_forward_kernel(int N, int V, T eps, const T* __restrict__ x, T* __restrict__ y) {
	const int n = blockIdx.x * blockDim.x + threadIdx.x;
	if (n >= N)
		return;
	T mx = x[n];
	for (int v = 1; v < V; ++v) {
		const T e = x[n + (size_t) N * v];
		mx = e > mx ? e : mx;
	}
	T s = (T) 0;
	for (int v = 0; v < V; ++v) {
		const T e = dev_exp(x[n + (size_t) N * v] - mx);
		y[n + (size_t) N * v] = e;
		s += e;
	}
	const T d = s + eps;
	for (int v = 0; v < V; ++v)
		y[n + (size_t) N * v] /= d;
}

/* dx_j = sum_i g_i (delta_ij y_i - y_i y_j) = y_j (g_j - sum_i g_i y_i) */
template<typename T>
__global__ void softmax_backward_kernel(int N, int V, const T* __restrict__ y, const T* __restrict__ g, T* __restrict__ dx) {
	const int n = blockIdx.x * blockDim.x + threadIdx.x;
	if (n >= N)
		return;
	T dot = (T) 0;
	for (int v = 0; v < V; ++v)
		dot += g[n + (size_t) N * v] * y[n + (size_t) N * v];
	for (int v = 0; v < V; ++v) {
		const size_t i = n + (size_t) N * v;
		dx[i] = y[i] * g[i] - y[i] * dot;
	}
}

/* ----------------------------------------------------------------------------------------------
 * PReLU / PSwish: per-activation parameter (1 x V), gradients are column sums over the batch
 * (layer/activation/PReLUActivationLayer.hpp:80-109, PSwishActivationLayer.hpp:77-99).
 * One wavefront per column for the backward pass.
 * -------------------------------------------------------------------------------------------- */
template<typename T, bool SWISH>
__global__ __launch_bounds__(256)
void param_act_forward_kernel(size_t total, int N, const T* __restrict__ param, const T* __restrict__ x, T* __restrict__ y) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
		const T p = param[i / N], xi = x[i];
		if (SWISH) {
			y[i] = xi * ((T) 1 / (dev_exp(xi * (-p)) + (T) 1));
		} else {
			const T ax = xi * p;
			y[i] = xi > ax ? xi : (ax == ax ? ax : xi);
		}
	}
}

template<typename T, bool SWISH>
__global__ __launch_bounds__(256)
void param_act_backward_kernel(int N, int V, const T* __restrict__ param, const T* __restrict__ x, const T* __restrict__ g,
		T* __restrict__ param_grad, T* __restrict__ dx) {
	const int v = blockIdx.x * 4 + threadIdx.x / 64;
	if (v >= V)
		return;
	const int lane = threadIdx.x % 64;
	const T p = param[v];
	T acc = (T) 0;
	for (int n = lane; n < N; n += 64) {
		const size_t i = n + (size_t) N * v;
		const T xi = x[i], gi = g[i];
		if (SWISH) {
			const T s = (T) 1 / (dev_exp(xi * (-p)) + (T) 1);
			acc += s * ((T) 1 - s) * xi * xi * gi;
			if (dx)
				dx[i] = s * ((((T) 1 - s) * p) * xi + (T) 1) * gi;
		} else {
			if (xi >= (T) 0) {
				if (dx)
					dx[i] = gi;
			} else {
				if (dx)
					dx[i] = p * gi;
				acc += xi * gi;
			}
		}
	}
	acc = wave_sum(acc);
	if (lane == 0)
		param_grad[v] += acc;
}

/* ----------------------------------------------------------------------------------------------
 * Batch norm (layer/BatchNormLayer.hpp:225-262 per channel, :411-456 per activation).
 * A statistics group is a contiguous slab of L elements. grid = (groups, splits); split s covers
 * [s*span, (s+1)*span) of the slab. Mean and variance (the mean of squared *centred* values, as in the
 * reference) come from one pass that merges per-thread, per-block and per-split moments in fixed orders.
 * -------------------------------------------------------------------------------------------- */
/* (count, mean, sum of squared deviations from the mean) of set b merged into those of set a (Chan, Golub,
 * LeVeque): exact in real arithmetic and as well conditioned as the two-pass formula, so the variance is the
 * mean of squared *centred* values, as in the reference, from a single read of the data. */
template<typename T>
__device__ __forceinline__ void moments_merge(T& n, T& mean, T& m2, T nb, T meanb, T m2b) {
	const T nt = n + nb;
	if (nt > (T) 0) {
		const T d = meanb - mean, w = nb / nt;
		mean += d * w;
		m2 += m2b + (d * d) * (n * w);
		n = nt;
	}
}

template<typename T, int V> struct SlabVec { typedef T type __attribute__((ext_vector_type(V))); };

/* Per-split moments of a slab: every thread merges groups of eight values (group mean, then centred squares,
 * both from registers), the 256 threads are merged pairwise in a fixed tree. V values per memory access;
 * for V > 1 the slab length, the span and the pointers are multiples of V values. */
template<typename T, int V>
__global__ __launch_bounds__(256)
void bn_moments_kernel(size_t L, size_t span, const T* __restrict__ x, T* __restrict__ ws_mean, T* __restrict__ ws_m2) {
	__shared__ T lds[3][256];
	constexpr int G = 8, NV = G / V;
	typedef typename SlabVec<T, V>::type vt;
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < L ? begin + span : L;
	const T* xs = x + (size_t) blockIdx.x * L;
	T n = (T) 0, mean = (T) 0, m2 = (T) 0;
	for (size_t i0 = begin + (size_t) threadIdx.x * V; i0 < end; i0 += (size_t) 256 * G) {
		T v[G];
		int cnt = 0;
		#pragma unroll
		for (int u = 0; u < NV; ++u) {
			const size_t i = i0 + (size_t) u * 256 * V;
			const bool in = i < end;
			vt a = {0};
			if (in)
				a = *reinterpret_cast<const vt*>(xs + i);
			#pragma unroll
			for (int e = 0; e < V; ++e)
				v[u * V + e] = a[e];
			cnt += in ? V : 0;
		}
		T sum = (T) 0;
		#pragma unroll
		for (int u = 0; u < G; ++u)
			sum += v[u];
		const T gm = sum / (T) cnt;
		T q = (T) 0;
		#pragma unroll
		for (int u = 0; u < G; ++u) {
			const T d = u < cnt ? v[u] - gm : (T) 0;        /* values past the end are the trailing ones */
			q += d * d;
		}
		moments_merge(n, mean, m2, (T) cnt, gm, q);
	}
	const int tid = threadIdx.x;
	lds[0][tid] = n;
	lds[1][tid] = mean;
	lds[2][tid] = m2;
	__syncthreads();
	for (int off = 128; off > 0; off >>= 1) {
		if (tid < off) {
			T a_n = lds[0][tid], a_mean = lds[1][tid], a_m2 = lds[2][tid];
			moments_merge(a_n, a_mean, a_m2, lds[0][tid + off], lds[1][tid + off], lds[2][tid + off]);
			lds[0][tid] = a_n;
			lds[1][tid] = a_mean;
			lds[2][tid] = a_m2;
		}
		__syncthreads();
	}
	if (tid == 0) {
		ws_mean[(size_t) blockIdx.x * gridDim.y + blockIdx.y] = lds[1][0];
		ws_m2[(size_t) blockIdx.x * gridDim.y + blockIdx.y] = lds[2][0];
	}
}

template<typename T>
__device__ __forceinline__ T sum_partials(const T* ws, int splits) {
	T s = (T) 0;
	for (int p = 0; p < splits; ++p)
		s += ws[p];
	return s;
}

/* Mean and biased variance of a slab from its per-split moments, merged in ascending order. */
template<typename T>
__device__ __forceinline__ void slab_moments(const T* ws_mean, const T* ws_m2, int splits, size_t L, size_t span, T& mean, T& var) {
	T n = (T) 0, m2 = (T) 0;
	mean = (T) 0;
	for (int p = 0; p < splits; ++p) {
		const size_t begin = (size_t) p * span;
		const size_t cnt = begin >= L ? 0 : (begin + span < L ? span : L - begin);
		moments_merge(n, mean, m2, (T) cnt, ws_mean[p], ws_m2[p]);
	}
	var = m2 / (T) L;
}

template<typename T, int V>
__global__ __launch_bounds__(256)
void bn_train_apply_kernel(size_t L, size_t span, const T* __restrict__ x, const T* __restrict__ gamma,
		const T* __restrict__ beta, T* __restrict__ avg_mean, T* __restrict__ avg_inv_sd, bool stats_init, T decay, T eps,
		const T* __restrict__ ws_sum, const T* __restrict__ ws_sq, T* __restrict__ out, T* __restrict__ std_cache,
		T* __restrict__ inv_sd_cache) {
	const int splits = gridDim.y;
	const int grp = blockIdx.x;
	T mean, var;
	slab_moments(ws_sum + (size_t) grp * splits, ws_sq + (size_t) grp * splits, splits, L, span, mean, var);
	const T inv_sd = (T) 1 / dev_sqrt(var + eps);
	const T ga = gamma[grp], be = beta[grp];
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < L ? begin + span : L;
	const T* xs = x + (size_t) grp * L;
	T* ys = out + (size_t) grp * L;
	T* sc = std_cache + (size_t) grp * L;
	typedef typename SlabVec<T, V>::type vt;
	for (size_t i = begin + (size_t) threadIdx.x * V; i < end; i += (size_t) 256 * V) {
		const vt xv = __builtin_nontemporal_load(reinterpret_cast<const vt*>(xs + i));
		vt sv, yv;
		#pragma unroll
		for (int e = 0; e < V; ++e) {
			sv[e] = (xv[e] - mean) * inv_sd;
			yv[e] = sv[e] * ga + be;
		}
		__builtin_nontemporal_store(sv, reinterpret_cast<vt*>(sc + i));
		__builtin_nontemporal_store(yv, reinterpret_cast<vt*>(ys + i));
	}
	if (blockIdx.y == 0 && threadIdx.x == 0) {
		inv_sd_cache[grp] = inv_sd;
		if (stats_init) {       /* running average (BatchNormLayer.hpp:234-238) */
			avg_mean[grp] = ((T) 1 - decay) * avg_mean[grp] + decay * mean;
			avg_inv_sd[grp] = ((T) 1 - decay) * avg_inv_sd[grp] + decay * inv_sd;
		} else {                /* first call assigns (:239-243) */
			avg_mean[grp] = mean;
			avg_inv_sd[grp] = inv_sd;
		}
	}
}

template<typename T, int V>
__global__ __launch_bounds__(256)
void bn_infer_kernel(size_t L, size_t span, const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
		const T* __restrict__ avg_mean, const T* __restrict__ avg_inv_sd, T* __restrict__ out) {
	const int grp = blockIdx.x;
	const T mean = avg_mean[grp], inv_sd = avg_inv_sd[grp], ga = gamma[grp], be = beta[grp];
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < L ? begin + span : L;
	const T* xs = x + (size_t) grp * L;
	T* ys = out + (size_t) grp * L;
	typedef typename SlabVec<T, V>::type vt;
	for (size_t i = begin + (size_t) threadIdx.x * V; i < end; i += (size_t) 256 * V) {
		const vt xv = __builtin_nontemporal_load(reinterpret_cast<const vt*>(xs + i));
		vt yv;
		#pragma unroll
		for (int e = 0; e < V; ++e)
			yv[e] = ((xv[e] - mean) * inv_sd) * ga + be;
		__builtin_nontemporal_store(yv, reinterpret_cast<vt*>(ys + i));
	}
}

template<typename T, int V>
__global__ __launch_bounds__(256)
void bn_backward_sums_kernel(size_t L, size_t span, const T* __restrict__ g, const T* __restrict__ std_cache,
		T* __restrict__ ws_g, T* __restrict__ ws_gs) {
	__shared__ T lds[4];
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < L ? begin + span : L;
	const T* gs = g + (size_t) blockIdx.x * L;
	const T* sc = std_cache + (size_t) blockIdx.x * L;
	typedef typename SlabVec<T, V>::type vt;
	constexpr int U = 4;        /* independent accesses in flight per thread and operand */
	T s1 = (T) 0, s2 = (T) 0;
	for (size_t i0 = begin + (size_t) threadIdx.x * V; i0 < end; i0 += (size_t) 256 * V * U) {
		vt gv[U], cv[U];
		#pragma unroll
		for (int u = 0; u < U; ++u) {
			const size_t i = i0 + (size_t) u * 256 * V;
			gv[u] = vt{0};
			cv[u] = vt{0};
			if (i < end) {
				gv[u] = *reinterpret_cast<const vt*>(gs + i);
				cv[u] = *reinterpret_cast<const vt*>(sc + i);
			}
		}
		#pragma unroll
		for (int u = 0; u < U; ++u) {
			#pragma unroll
			for (int e = 0; e < V; ++e) {
				s1 += gv[u][e];
				s2 += gv[u][e] * cv[u][e];
			}
		}
	}
	s1 = block_sum_256(s1, lds);
	s2 = block_sum_256(s2, lds);
	if (threadIdx.x == 0) {
		ws_g[(size_t) blockIdx.x * gridDim.y + blockIdx.y] = s1;
		ws_gs[(size_t) blockIdx.x * gridDim.y + blockIdx.y] = s2;
	}
}

template<typename T, int V>
__global__ __launch_bounds__(256)
void bn_backward_apply_kernel(size_t L, size_t span, const T* __restrict__ g, const T* __restrict__ gamma,
		const T* __restrict__ std_cache, const T* __restrict__ inv_sd_cache, const T* __restrict__ ws_g,
		const T* __restrict__ ws_gs, T* __restrict__ gamma_grad, T* __restrict__ beta_grad, T* __restrict__ in_grad) {
	const int splits = gridDim.y;
	const int grp = blockIdx.x;
	const T sum_g = sum_partials(ws_g + (size_t) grp * splits, splits);
	const T sum_gs = sum_partials(ws_gs + (size_t) grp * splits, splits);
	if (blockIdx.y == 0 && threadIdx.x == 0) {
		gamma_grad[grp] += sum_gs;          /* BatchNormLayer.hpp:252-253 */
		beta_grad[grp] += sum_g;            /* :254 */
	}
	if (!in_grad)
		return;
	const T ga = gamma[grp];
	const T sum_sg = sum_g * ga, sum_ssg = sum_gs * ga;       /* sums of g*gamma and of std_in * g*gamma */
	const T scale = ((T) 1 / (T) L) * inv_sd_cache[grp];      /* :260-261 */
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < L ? begin + span : L;
	const T* gs = g + (size_t) grp * L;
	const T* sc = std_cache + (size_t) grp * L;
	T* dx = in_grad + (size_t) grp * L;
	typedef typename SlabVec<T, V>::type vt;
	for (size_t i = begin + (size_t) threadIdx.x * V; i < end; i += (size_t) 256 * V) {
		const vt gv = __builtin_nontemporal_load(reinterpret_cast<const vt*>(gs + i));
		const vt cv = __builtin_nontemporal_load(reinterpret_cast<const vt*>(sc + i));
		vt o;
		#pragma unroll
		for (int e = 0; e < V; ++e)
			o[e] = (((T) L * (gv[e] * ga) - sum_sg) - cv[e] * sum_ssg) * scale;
		__builtin_nontemporal_store(o, reinterpret_cast<vt*>(dx + i));
	}
}

constexpr int BN_MAX_SPLITS = 64;

int bn_splits(int groups, size_t L) {
	const size_t by_len = std::max<size_t>(1, L / 2048);
	const size_t by_fill = std::max<size_t>(1, (size_t) 2048 / (size_t) std::max(1, groups));
	return (int) std::min<size_t>(BN_MAX_SPLITS, std::min(by_len, by_fill));
}

/* ----------------------------------------------------------------------------------------------
 * Pooling (layer/PoolLayer.hpp:77-116, layer/pool/MaxPoolLayer.hpp:38-80, MeanPoolLayer.hpp:35-41).
 * One thread per output element (forward) or per input element (backward, gather form: each
 * input sums the windows that cover it in the reference's patch order, so overlapping windows
 * accumulate without atomics and in the reference's order of additions).
 * -------------------------------------------------------------------------------------------- */
/* Thread layout of the pooling kernels: a thread owns VN consecutive samples (one 16-byte access when
 * the batch allows it) of POOL_ROWS rows; a block is TX such threads wide and 256/TX tall. Rows are
 * output rows in the forward pass and input rows in the backward pass. The block index carries
 * (channel, column, row block, sample block), decoded with block-uniform scalar arithmetic. */
constexpr int POOL_ROWS = 4;

struct PoolLaunch {
	int tx, ty, nblks, rblks;
};

template<typename T, int VN>
__device__ __forceinline__ void pool_load(T (&dst)[VN], const T* p) {
	if constexpr (VN == 1) {
		dst[0] = *p;
	} else {
		typedef T vt __attribute__((ext_vector_type(VN)));
		const vt v = *reinterpret_cast<const vt*>(p);
		#pragma unroll
		for (int i = 0; i < VN; ++i)
			dst[i] = v[i];
	}
}

template<typename T, int VN>
__device__ __forceinline__ void pool_store(T* p, const T (&src)[VN]) {
	if constexpr (VN == 1) {
		*p = src[0];
	} else {
		typedef T vt __attribute__((ext_vector_type(VN)));
		vt v;
		#pragma unroll
		for (int i = 0; i < VN; ++i)
			v[i] = src[i];
		__builtin_nontemporal_store(v, reinterpret_cast<vt*>(p));
	}
}

template<typename T, bool MAX, int VN>
__global__ __launch_bounds__(256)
void pool_forward_kernel(PoolShape s, int N, int OH, int OW, PoolLaunch pl, const T* __restrict__ x, T* __restrict__ out,
		unsigned* __restrict__ inds) {
	unsigned b = blockIdx.x;
	const int nb = (int) (b % (unsigned) pl.nblks);
	b /= (unsigned) pl.nblks;
	const int rb = (int) (b % (unsigned) pl.rblks);
	b /= (unsigned) pl.rblks;
	const int ow = (int) (b % (unsigned) OW);
	const int c = (int) (b / (unsigned) OW);
	const int n = (nb * pl.tx + (int) threadIdx.x % pl.tx) * VN;
	if (n >= N)
		return;
	const int row0 = rb * pl.ty * POOL_ROWS + (int) threadIdx.x / pl.tx;
	#pragma unroll
	for (int j = 0; j < POOL_ROWS; ++j) {
		const int oh = row0 + j * pl.ty;
		if (oh >= OH)
			break;
		const T* base = x + n + (size_t) N * ((size_t) oh * s.sv + (size_t) s.H * ((size_t) ow * s.sh + (size_t) s.W * c));
		const size_t oidx = n + (size_t) N * (oh + (size_t) OH * (ow + (size_t) OW * c));
		T res[VN];
		if (MAX) {
			/* strict '>' from lowest(): first maximum in (width-major, height-minor) order wins and NaN
			 * is never selected (MaxPoolLayer.hpp:45-56) */
			unsigned bi[VN];
			#pragma unroll
			for (int v = 0; v < VN; ++v) {
				res[v] = std::numeric_limits<T>::lowest();
				bi[v] = 0;
			}
			for (int k = 0; k < s.RW; ++k)
				for (int l = 0; l < s.RH; ++l) {
					T val[VN];
					pool_load<T, VN>(val, base + (size_t) N * (l + (size_t) s.H * k));
					#pragma unroll
					for (int v = 0; v < VN; ++v)
						if (val[v] > res[v]) {
							res[v] = val[v];
							bi[v] = (unsigned) (k * s.RH + l);
						}
				}
			pool_store<unsigned, VN>(inds + (((size_t) ow * OH + oh) * ((size_t) s.C * N) + (size_t) c * N + n), bi);
		} else {
			#pragma unroll
			for (int v = 0; v < VN; ++v)
				res[v] = (T) 0;
			for (int k = 0; k < s.RW; ++k)
				for (int l = 0; l < s.RH; ++l) {
					T val[VN];
					pool_load<T, VN>(val, base + (size_t) N * (l + (size_t) s.H * k));
					#pragma unroll
					for (int v = 0; v < VN; ++v)
						res[v] += val[v];
				}
			#pragma unroll
			for (int v = 0; v < VN; ++v)
				res[v] = res[v] / (T) (s.RH * s.RW);
		}
		pool_store<T, VN>(out + oidx, res);
	}
}

template<typename T, bool MAX, int VN>
__global__ __launch_bounds__(256)
void pool_backward_kernel(PoolShape s, int N, int OH, int OW, PoolLaunch pl, const T* __restrict__ g,
		const unsigned* __restrict__ inds, T* __restrict__ dx) {
	unsigned b = blockIdx.x;
	const int nb = (int) (b % (unsigned) pl.nblks);
	b /= (unsigned) pl.nblks;
	const int rb = (int) (b % (unsigned) pl.rblks);
	b /= (unsigned) pl.rblks;
	const int w = (int) (b % (unsigned) s.W);
	const int c = (int) (b / (unsigned) s.W);
	const int n = (nb * pl.tx + (int) threadIdx.x % pl.tx) * VN;
	if (n >= N)
		return;
	/* windows [o*stride, o*stride + R) containing the coordinate; the column range is block-uniform */
	const int ow_lo = w >= s.RW ? (w - s.RW + s.sh) / s.sh : 0;
	const int ow_hi = min(w / s.sh, OW - 1);
	const T area = (T) (s.RH * s.RW);
	const int row0 = rb * pl.ty * POOL_ROWS + (int) threadIdx.x / pl.tx;
	#pragma unroll
	for (int j = 0; j < POOL_ROWS; ++j) {
		const int h = row0 + j * pl.ty;
		if (h >= s.H)
			break;
		const int oh_lo = h >= s.RH ? (h - s.RH + s.sv) / s.sv : 0;
		const int oh_hi = min(h / s.sv, OH - 1);
		T sum[VN];
		#pragma unroll
		for (int v = 0; v < VN; ++v)
			sum[v] = (T) 0;
		for (int ow = ow_lo; ow <= ow_hi; ++ow)
			for (int oh = oh_lo; oh <= oh_hi; ++oh) {
				T gv[VN];
				pool_load<T, VN>(gv, g + (n + (size_t) N * (oh + (size_t) OH * (ow + (size_t) OW * c))));
				if (MAX) {
					unsigned ind[VN];
					pool_load<unsigned, VN>(ind, inds + (((size_t) ow * OH + oh) * ((size_t) s.C * N) + (size_t) c * N + n));
					const unsigned mine = (unsigned) (w - ow * s.sh) * (unsigned) s.RH + (unsigned) (h - oh * s.sv);
					#pragma unroll
					for (int v = 0; v < VN; ++v)
						sum[v] += ind[v] == mine ? gv[v] : (T) 0;
				} else {
					#pragma unroll
					for (int v = 0; v < VN; ++v)
						sum[v] += gv[v] / area;
				}
			}
		pool_store<T, VN>(dx + (n + (size_t) N * (h + (size_t) s.H * (w + (size_t) s.W * c))), sum);
	}
}

/* Backward pass when the windows tile the input exactly (stride = receptor, no rows or columns left over): every
 * input position belongs to one window, so a thread takes one window, reads its upstream gradient (and argmax)
 * once and writes the window's RH x RW input gradients. Same values as the gather form. */
template<typename T, bool MAX, int VN>
__global__ __launch_bounds__(256)
void pool_backward_tiled_kernel(PoolShape s, int N, int OH, int OW, PoolLaunch pl, const T* __restrict__ g,
		const unsigned* __restrict__ inds, T* __restrict__ dx) {
	unsigned b = blockIdx.x;
	const int nb = (int) (b % (unsigned) pl.nblks);
	b /= (unsigned) pl.nblks;
	const int rb = (int) (b % (unsigned) pl.rblks);
	b /= (unsigned) pl.rblks;
	const int ow = (int) (b % (unsigned) OW);
	const int c = (int) (b / (unsigned) OW);
	const int n = (nb * pl.tx + (int) threadIdx.x % pl.tx) * VN;
	if (n >= N)
		return;
	const T area = (T) (s.RH * s.RW);
	const int row0 = rb * pl.ty * POOL_ROWS + (int) threadIdx.x / pl.tx;
	#pragma unroll
	for (int j = 0; j < POOL_ROWS; ++j) {
		const int oh = row0 + j * pl.ty;
		if (oh >= OH)
			break;
		T gv[VN];
		unsigned ind[VN];
		pool_load<T, VN>(gv, g + (n + (size_t) N * (oh + (size_t) OH * (ow + (size_t) OW * c))));
		if (MAX)
			pool_load<unsigned, VN>(ind, inds + (((size_t) ow * OH + oh) * ((size_t) s.C * N) + (size_t) c * N + n));
		T* base = dx + n + (size_t) N * ((size_t) oh * s.RH + (size_t) s.H * ((size_t) ow * s.RW + (size_t) s.W * c));
		for (int k = 0; k < s.RW; ++k)
			for (int l = 0; l < s.RH; ++l) {
				T o[VN];
				#pragma unroll
				for (int v = 0; v < VN; ++v)
					o[v] = MAX ? (ind[v] == (unsigned) (k * s.RH + l) ? (T) 0 + gv[v] : (T) 0) : (T) 0 + gv[v] / area;
				pool_store<T, VN>(base + (size_t) N * (l + (size_t) s.H * k), o);
			}
	}
}

/* vn = samples per thread */
PoolLaunch pool_launch(int N, int rows, int vn) {
	const int nthreads = (N + vn - 1) / vn;
	PoolLaunch pl;
	pl.tx = 256;
	while (pl.tx > 1 && pl.tx / 2 >= nthreads)
		pl.tx /= 2;
	pl.ty = 256 / pl.tx;
	pl.nblks = (nthreads + pl.tx - 1) / pl.tx;
	pl.rblks = (rows + pl.ty * POOL_ROWS - 1) / (pl.ty * POOL_ROWS);
	return pl;
}

unsigned pool_grid(const PoolLaunch& pl, int cols, int channels) {
	const double blocks = (double) pl.nblks * pl.rblks * cols * channels;
	CATTLE_HIP_REQUIRE(blocks < 2147483647.0, "pooling launch exceeds the grid limit");
	return (unsigned) blocks;
}

/* Zero fill of `bytes` bytes at a 4-byte aligned address: 16-byte stores over the aligned middle, 4-byte stores over
 * the ends. A kernel rather than a memset of the runtime, so that the call may be recorded into a graph. */
__global__ __launch_bounds__(256)
void zero_fill_kernel(unsigned* __restrict__ p, size_t words) {
	const size_t head = std::min<size_t>(words, (size_t) ((16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15) / 4);
	const size_t quads = (words - head) / 4;
	uint4* q = reinterpret_cast<uint4*>(p + head);
	const size_t stride = (size_t) gridDim.x * blockDim.x, t = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
	for (size_t i = t; i < quads; i += stride)
		q[i] = make_uint4(0u, 0u, 0u, 0u);
	if (t < head)
		p[t] = 0u;
	const size_t done = head + quads * 4;
	if (t < words - done)
		p[done + t] = 0u;
}

template<typename T>
__global__ void axpy_one_kernel(size_t n, const T* __restrict__ src, T* __restrict__ dst) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
		dst[i] += src[i];
}

/* ----------------------------------------------------------------------------------------------
 * Small matrix helpers of the transposed convolution: its weight matrix is the transpose of the
 * equivalent convolution's, and its bias has one entry per output activation
 * (layer/kernel/TransConvKernelLayer.hpp:46-56, :143-144, :153-155).
 * -------------------------------------------------------------------------------------------- */
template<typename T, bool ACC>
__global__ __launch_bounds__(256)
void transpose_kernel(int rows, int cols, const T* __restrict__ src, T* __restrict__ dst) {
	__shared__ T tile[32][33];
	const int r0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
	const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
	for (int j = ty; j < 32; j += 8) {
		const int r = r0 + tx, c = c0 + j;
		tile[j][tx] = r < rows && c < cols ? src[(size_t) r + (size_t) rows * c] : (T) 0;
	}
	__syncthreads();
	for (int j = ty; j < 32; j += 8) {
		const int c = c0 + tx, r = r0 + j;
		if (r < rows && c < cols) {
			const size_t o = (size_t) c + (size_t) cols * r;
			dst[o] = ACC ? dst[o] + tile[tx][j] : tile[tx][j];
		}
	}
}

template<typename T>
__global__ __launch_bounds__(256)
void add_row_vector_kernel(size_t total, int N, const T* __restrict__ row, T* __restrict__ x) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
		x[i] += row[i / (size_t) N];
}

/* one wavefront per column: lanes stride over the N contiguous entries, fixed-order shuffle sum */
template<typename T>
__global__ __launch_bounds__(256)
void column_sums_kernel(int N, size_t V, const T* __restrict__ x, T* __restrict__ row) {
	const int lane = threadIdx.x % 64;
	const size_t waves = (size_t) gridDim.x * 4;
	for (size_t e = (size_t) blockIdx.x * 4 + threadIdx.x / 64; e < V; e += waves) {
		T s = (T) 0;
		for (int n = lane; n < N; n += 64)
			s += x[(size_t) n + (size_t) N * e];
		s = wave_sum(s);
		if (lane == 0)
			row[e] += s;
	}
}

/* ----------------------------------------------------------------------------------------------
 * LSTM cell arithmetic between the kernel layers (lstm_math.hpp), one thread per state element.
 * -------------------------------------------------------------------------------------------- */
template<typename T>
__global__ __launch_bounds__(256)
void lstm_gates_forward_kernel(const LstmForwardStep<T> A, const T* __restrict__ zh) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t e = (size_t) blockIdx.x * blockDim.x + threadIdx.x; e < A.P; e += stride) {
		T zh4[4];       /* (assigned on every path: a partly initialised register array ends up in scratch memory) */
		#pragma unroll
		for (int g = 0; g < 4; ++g)
			zh4[g] = zh ? zh[g * A.P + e] : (T) 0;
		if (lstm_standard_acts(A.a))
			lstm_forward_element<T, true>(A, (unsigned) e, zh != nullptr, zh4);
		else
			lstm_forward_element<T, false>(A, (unsigned) e, zh != nullptr, zh4);
	}
}

template<typename T>
__global__ __launch_bounds__(256)
void lstm_gates_backward_kernel(const LstmBackwardStep<T> A, const T* __restrict__ dh) {
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	for (size_t e = (size_t) blockIdx.x * blockDim.x + threadIdx.x; e < A.P; e += stride) {
		if (lstm_standard_acts(A.a))
			lstm_backward_element<T, true>(A, (unsigned) e, dh != nullptr, dh ? dh[e] : (T) 0);
		else
			lstm_backward_element<T, false>(A, (unsigned) e, dh != nullptr, dh ? dh[e] : (T) 0);
	}
}

void check_launch() {
	CATTLE_HIP_CHECK(hipGetLastError());
}

} /* namespace */

template<typename T>
void act_forward(int kind, size_t n, T p, const T* x, T* y) {
	if (n == 0)
		return;
	switch (kind) {
	case ACT_IDENTITY: act_forward_kind<T, ACT_IDENTITY>(n, p, x, y); break;
	case ACT_SCALED: act_forward_kind<T, ACT_SCALED>(n, p, x, y); break;
	case ACT_BINARY_STEP: act_forward_kind<T, ACT_BINARY_STEP>(n, p, x, y); break;
	case ACT_SIGMOID: act_forward_kind<T, ACT_SIGMOID>(n, p, x, y); break;
	case ACT_TANH: act_forward_kind<T, ACT_TANH>(n, p, x, y); break;
	case ACT_SOFTSIGN: act_forward_kind<T, ACT_SOFTSIGN>(n, p, x, y); break;
	case ACT_SOFTPLUS: act_forward_kind<T, ACT_SOFTPLUS>(n, p, x, y); break;
	case ACT_RELU: act_forward_kind<T, ACT_RELU>(n, p, x, y); break;
	case ACT_LEAKY_RELU: act_forward_kind<T, ACT_LEAKY_RELU>(n, p, x, y); break;
	case ACT_ELU: act_forward_kind<T, ACT_ELU>(n, p, x, y); break;
	case ACT_SWISH: act_forward_kind<T, ACT_SWISH>(n, p, x, y); break;
	default: throw Error(ERR_INVALID, "unknown activation kind");
	}
	check_launch();
}

template<typename T>
void act_backward(int kind, size_t n, T p, const T* x, const T* y, const T* g, T* dx) {
	if (n == 0)
		return;
	switch (kind) {
	case ACT_IDENTITY: act_backward_kind<T, ACT_IDENTITY>(n, p, x, y, g, dx); break;
	case ACT_SCALED: act_backward_kind<T, ACT_SCALED>(n, p, x, y, g, dx); break;
	case ACT_BINARY_STEP: act_backward_kind<T, ACT_BINARY_STEP>(n, p, x, y, g, dx); break;
	case ACT_SIGMOID: act_backward_kind<T, ACT_SIGMOID>(n, p, x, y, g, dx); break;
	case ACT_TANH: act_backward_kind<T, ACT_TANH>(n, p, x, y, g, dx); break;
	case ACT_SOFTSIGN: act_backward_kind<T, ACT_SOFTSIGN>(n, p, x, y, g, dx); break;
	case ACT_SOFTPLUS: act_backward_kind<T, ACT_SOFTPLUS>(n, p, x, y, g, dx); break;
	case ACT_RELU: act_backward_kind<T, ACT_RELU>(n, p, x, y, g, dx); break;
	case ACT_LEAKY_RELU: act_backward_kind<T, ACT_LEAKY_RELU>(n, p, x, y, g, dx); break;
	case ACT_ELU: act_backward_kind<T, ACT_ELU>(n, p, x, y, g, dx); break;
	case ACT_SWISH: act_backward_kind<T, ACT_SWISH>(n, p, x, y, g, dx); break;
	default: throw Error(ERR_INVALID, "unknown activation kind");
	}
	check_launch();
}

template<typename T>
void softmax_forward(int N, int V, T eps, const T* x, T* y) {
	softmax_forward_kernel<T><<<(unsigned) ((N + 63) / 64), 64, 0, stream()>>>(N, V, eps, x, y);
	check_launch();
}

template<typename T>
void softmax_backward(int N, int V, const T* y, const T* g, T* dx) {
	softmax_backward_kernel<T><<<(unsigned) ((N + 63) / 64), 64, 0, stream()>>>(N, V, y, g, dx);
	check_launch();
}

template<typename T>
void prelu_forward(int N, int V, const T* alpha, const T* x, T* y) {
	const size_t total = (size_t) N * V;
	param_act_forward_kernel<T, false><<<stream_grid(total), 256, 0, stream()>>>(total, N, alpha, x, y);
	check_launch();
}

template<typename T>
void prelu_backward(int N, int V, const T* alpha, const T* x, const T* g, T* alpha_grad, T* dx) {
	param_act_backward_kernel<T, false><<<(unsigned) ((V + 3) / 4), 256, 0, stream()>>>(N, V, alpha, x, g, alpha_grad, dx);
	check_launch();
}

template<typename T>
void pswish_forward(int N, int V, const T* beta, const T* x, T* y) {
	const size_t total = (size_t) N * V;
	param_act_forward_kernel<T, true><<<stream_grid(total), 256, 0, stream()>>>(total, N, beta, x, y);
	check_launch();
}

template<typename T>
void pswish_backward(int N, int V, const T* beta, const T* x, const T* g, T* beta_grad, T* dx) {
	param_act_backward_kernel<T, true><<<(unsigned) ((V + 3) / 4), 256, 0, stream()>>>(N, V, beta, x, g, beta_grad, dx);
	check_launch();
}

size_t bn_workspace(int groups, size_t L) {
	(void) L;
	return (size_t) 2 * groups * BN_MAX_SPLITS;
}

/* The span of a split is a multiple of four values, so that 16-byte accesses stay aligned within a slab. */
size_t bn_span(size_t L, int splits) {
	const size_t span = (L + splits - 1) / splits;
	return (span + 3) / 4 * 4;
}

template<typename T, int V>
void bn_forward_launch(int groups, size_t L, const T* x, const T* gamma, const T* beta, T* avg_mean, T* avg_inv_sd,
		bool stats_init, bool training, T decay, T eps, T* out, T* std_cache, T* inv_sd_cache, T* ws) {
	const int splits = bn_splits(groups, L);
	const size_t span = bn_span(L, splits);
	dim3 grid((unsigned) groups, (unsigned) splits);
	if (training) {
		T* ws_sum = ws;
		T* ws_sq = ws + (size_t) groups * BN_MAX_SPLITS;
		bn_moments_kernel<T, V><<<grid, 256, 0, stream()>>>(L, span, x, ws_sum, ws_sq);
		check_launch();
		bn_train_apply_kernel<T, V><<<grid, 256, 0, stream()>>>(L, span, x, gamma, beta, avg_mean, avg_inv_sd, stats_init, decay,
				eps, ws_sum, ws_sq, out, std_cache, inv_sd_cache);
		check_launch();
	} else {
		bn_infer_kernel<T, V><<<grid, 256, 0, stream()>>>(L, span, x, gamma, beta, avg_mean, avg_inv_sd, out);
		check_launch();
	}
}

template<typename T>
void bn_forward(int groups, size_t L, const T* x, const T* gamma, const T* beta, T* avg_mean, T* avg_inv_sd,
		bool stats_init, bool training, T decay, T eps, T* out, T* std_cache, T* inv_sd_cache, T* ws) {
	constexpr int V = Pack<T>::V;
	if (L % V == 0 && aligned16(x) && aligned16(out) && (!training || aligned16(std_cache)))
		bn_forward_launch<T, V>(groups, L, x, gamma, beta, avg_mean, avg_inv_sd, stats_init, training, decay, eps, out, std_cache,
				inv_sd_cache, ws);
	else
		bn_forward_launch<T, 1>(groups, L, x, gamma, beta, avg_mean, avg_inv_sd, stats_init, training, decay, eps, out, std_cache,
				inv_sd_cache, ws);
}

template<typename T, int V>
void bn_backward_launch(int groups, size_t L, const T* out_grad, const T* gamma, const T* std_cache, const T* inv_sd_cache,
		T* gamma_grad, T* beta_grad, T* in_grad, T* ws) {
	const int splits = bn_splits(groups, L);
	const size_t span = bn_span(L, splits);
	dim3 grid((unsigned) groups, (unsigned) splits);
	T* ws_g = ws;
	T* ws_gs = ws + (size_t) groups * BN_MAX_SPLITS;
	bn_backward_sums_kernel<T, V><<<grid, 256, 0, stream()>>>(L, span, out_grad, std_cache, ws_g, ws_gs);
	check_launch();
	bn_backward_apply_kernel<T, V><<<grid, 256, 0, stream()>>>(L, span, out_grad, gamma, std_cache, inv_sd_cache, ws_g, ws_gs,
			gamma_grad, beta_grad, in_grad);
	check_launch();
}

template<typename T>
void bn_backward(int groups, size_t L, const T* out_grad, const T* gamma, const T* std_cache, const T* inv_sd_cache,
		T* gamma_grad, T* beta_grad, T* in_grad, T* ws) {
	constexpr int V = Pack<T>::V;
	if (L % V == 0 && aligned16(out_grad) && aligned16(std_cache) && (!in_grad || aligned16(in_grad)))
		bn_backward_launch<T, V>(groups, L, out_grad, gamma, std_cache, inv_sd_cache, gamma_grad, beta_grad, in_grad, ws);
	else
		bn_backward_launch<T, 1>(groups, L, out_grad, gamma, std_cache, inv_sd_cache, gamma_grad, beta_grad, in_grad, ws);
}

/* float tensors use 4 samples per thread (16-byte accesses) when possible; doubles use 2 */
template<typename T, bool MAX>
void pool_forward_launch(const PoolShape& s, int N, const T* x, T* out, unsigned* inds) {
	constexpr int VN = 16 / (int) sizeof(T);
	if (N % 4 == 0 && aligned16(x) && aligned16(out) && (!inds || aligned16(inds))) {
		const PoolLaunch pl = pool_launch(N, s.OH(), VN);
		pool_forward_kernel<T, MAX, VN><<<pool_grid(pl, s.OW(), s.C), 256, 0, stream()>>>(s, N, s.OH(), s.OW(), pl, x, out, inds);
	} else {
		const PoolLaunch pl = pool_launch(N, s.OH(), 1);
		pool_forward_kernel<T, MAX, 1><<<pool_grid(pl, s.OW(), s.C), 256, 0, stream()>>>(s, N, s.OH(), s.OW(), pl, x, out, inds);
	}
	check_launch();
}

template<typename T, bool MAX>
void pool_backward_launch(const PoolShape& s, int N, const T* out_grad, const unsigned* inds, T* in_grad) {
	constexpr int VN = 16 / (int) sizeof(T);
	const bool vec = N % 4 == 0 && aligned16(out_grad) && aligned16(in_grad) && (!inds || aligned16(inds));
	if (s.sv == s.RH && s.sh == s.RW && s.OH() * s.RH == s.H && s.OW() * s.RW == s.W) {
		if (vec) {
			const PoolLaunch pl = pool_launch(N, s.OH(), VN);
			pool_backward_tiled_kernel<T, MAX, VN><<<pool_grid(pl, s.OW(), s.C), 256, 0, stream()>>>(s, N, s.OH(), s.OW(), pl,
					out_grad, inds, in_grad);
		} else {
			const PoolLaunch pl = pool_launch(N, s.OH(), 1);
			pool_backward_tiled_kernel<T, MAX, 1><<<pool_grid(pl, s.OW(), s.C), 256, 0, stream()>>>(s, N, s.OH(), s.OW(), pl,
					out_grad, inds, in_grad);
		}
		check_launch();
		return;
	}
	if (vec) {
		const PoolLaunch pl = pool_launch(N, s.H, VN);
		pool_backward_kernel<T, MAX, VN><<<pool_grid(pl, s.W, s.C), 256, 0, stream()>>>(s, N, s.OH(), s.OW(), pl, out_grad, inds,
				in_grad);
	} else {
		const PoolLaunch pl = pool_launch(N, s.H, 1);
		pool_backward_kernel<T, MAX, 1><<<pool_grid(pl, s.W, s.C), 256, 0, stream()>>>(s, N, s.OH(), s.OW(), pl, out_grad, inds,
				in_grad);
	}
	check_launch();
}

template<typename T>
void maxpool_forward(const PoolShape& s, int N, const T* x, T* out, unsigned* inds) {
	pool_forward_launch<T, true>(s, N, x, out, inds);
}

template<typename T>
void maxpool_backward(const PoolShape& s, int N, const T* out_grad, const unsigned* inds, T* in_grad) {
	pool_backward_launch<T, true>(s, N, out_grad, inds, in_grad);
}

template<typename T>
void meanpool_forward(const PoolShape& s, int N, const T* x, T* out) {
	pool_forward_launch<T, false>(s, N, x, out, nullptr);
}

template<typename T>
void meanpool_backward(const PoolShape& s, int N, const T* out_grad, T* in_grad) {
	pool_backward_launch<T, false>(s, N, out_grad, nullptr, in_grad);
}

void device_zero_fill(void* dst, size_t bytes) {
	if (bytes == 0)
		return;
	CATTLE_HIP_REQUIRE((reinterpret_cast<uintptr_t>(dst) & 3) == 0 && bytes % 4 == 0, "zero fill of a buffer that is not made of 4-byte words");
	const size_t words = bytes / 4;
	const size_t blocks = std::min<size_t>(std::max<size_t>(1, (words / 4 + 255) / 256), 2048);
	zero_fill_kernel<<<(unsigned) blocks, 256, 0, stream()>>>(static_cast<unsigned*>(dst), words);
	check_launch();
}

template<typename T>
void axpy_one(size_t n, const T* src, T* dst) {
	if (n == 0)
		return;
	axpy_one_kernel<T><<<stream_grid(n), 256, 0, stream()>>>(n, src, dst);
	check_launch();
}

template<typename T>
void transpose_matrix(int rows, int cols, const T* src, T* dst, bool accumulate) {
	if (rows == 0 || cols == 0)
		return;
	const dim3 grid((unsigned) ((rows + 31) / 32), (unsigned) ((cols + 31) / 32));
	if (accumulate)
		transpose_kernel<T, true><<<grid, 256, 0, stream()>>>(rows, cols, src, dst);
	else
		transpose_kernel<T, false><<<grid, 256, 0, stream()>>>(rows, cols, src, dst);
	check_launch();
}

template<typename T>
void add_row_vector(int N, size_t V, const T* row, T* x) {
	const size_t total = (size_t) N * V;
	if (total == 0)
		return;
	add_row_vector_kernel<T><<<stream_grid(total), 256, 0, stream()>>>(total, N, row, x);
	check_launch();
}

template<typename T>
void accumulate_column_sums(int N, size_t V, const T* x, T* row) {
	if (V == 0 || N == 0)
		return;
	const size_t blocks = std::min<size_t>((V + 3) / 4, 256 * 16);
	column_sums_kernel<T><<<(unsigned) blocks, 256, 0, stream()>>>(N, V, x, row);
	check_launch();
}

template<typename T>
void lstm_gates_forward(const LstmForwardStep<T>& A, const T* zh) {
	if (A.P == 0)
		return;
	CATTLE_HIP_REQUIRE(A.P % (size_t) A.N == 0 && A.P <= 0x3fffffffu, "LSTM slab: whole samples, at most 2^30 elements");
	lstm_gates_forward_kernel<T><<<stream_grid(A.P), 256, 0, stream()>>>(A, zh);
	check_launch();
}

template<typename T>
void lstm_gates_backward(const LstmBackwardStep<T>& A, const T* dh) {
	if (A.P == 0)
		return;
	CATTLE_HIP_REQUIRE(A.P % (size_t) A.N == 0 && A.P <= 0x3fffffffu, "LSTM slab: whole samples, at most 2^30 elements");
	CATTLE_HIP_REQUIRE((A.zx_fwd == nullptr) == (A.zh_fwd == nullptr), "multiplicative integration needs both weighted tensors");
	lstm_gates_backward_kernel<T><<<stream_grid(A.P), 256, 0, stream()>>>(A, dh);
	check_launch();
}

/* ---- DropoutLayer (layer/DropoutLayer.hpp:74-96) ------------------------------------------------
 * y = x * mask, mask = (u <= dropout_prob ? 0 : 1 / (1 - dropout_prob + epsilon)); the backward pass is the
 * same product on the output gradient. The mask is never stored: both passes regenerate u from the pass key,
 * which leaves 8 bytes of traffic per element and pass (fp32). The uniform numbers are outputs of splitmix64
 * (Steele, Lea, Flood 2014) seeded with the key: a double takes the top 53 bits of output i, a float 24 bits of
 * output i / 2 (bits 63..40 for even i, bits 31..8 for odd i), i being the linear index in the batch tensor. */
typedef unsigned long long u64;

namespace {

__host__ __device__ __forceinline__ u64 splitmix64_output(u64 seed, u64 index) {
	u64 z = seed + (index + 1) * 0x9E3779B97F4A7C15ull;
	z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
	z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
	return z ^ (z >> 31);
}

__device__ __forceinline__ float dropout_uniform(u64 key, u64 i, float) {
	const u64 bits = splitmix64_output(key, i >> 1);
	return (float) (unsigned) ((i & 1) ? (bits >> 8) & 0xFFFFFFull : bits >> 40) * (1.0f / 16777216.0f);
}
__device__ __forceinline__ double dropout_uniform(u64 key, u64 i, double) {
	return (double) (splitmix64_output(key, i) >> 11) * (1.0 / 9007199254740992.0);
}

template<typename T, bool VECTOR>
__global__ __launch_bounds__(256)
void dropout_kernel(size_t n, u64 key, T prob, T scaling_factor, const T* __restrict__ x, T* __restrict__ y) {
	constexpr int V = VECTOR ? Pack<T>::V : 1;
	typedef typename Pack<T>::type vt;
	const size_t stride = (size_t) gridDim.x * blockDim.x;
	const size_t nv = n / V;
	for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
		if constexpr (VECTOR) {
			const vt a = __builtin_nontemporal_load(reinterpret_cast<const vt*>(x) + i);
			vt o;
			#pragma unroll
			for (int e = 0; e < V; ++e)
				o[e] = a[e] * (dropout_uniform(key, (u64) i * V + e, T()) <= prob ? (T) 0 : scaling_factor);
			__builtin_nontemporal_store(o, reinterpret_cast<vt*>(y) + i);
		} else {
			y[i] = x[i] * (dropout_uniform(key, (u64) i, T()) <= prob ? (T) 0 : scaling_factor);
		}
	}
	if (VECTOR && blockIdx.x == 0 && threadIdx.x < n - nv * V) {
		const size_t i = nv * V + threadIdx.x;
		y[i] = x[i] * (dropout_uniform(key, (u64) i, T()) <= prob ? (T) 0 : scaling_factor);
	}
}

} /* namespace */

u64 dropout_pass_key(u64 seed, u64 pass) {
	return splitmix64_output(seed, pass);
}

template<typename T>
void dropout_apply(size_t n, u64 key, T prob, T eps, const T* x, T* y) {
	if (n == 0)
		return;
	const T scaling_factor = (T) 1 / ((T) 1 - prob + eps);
	if (aligned16(x) && aligned16(y))
		dropout_kernel<T, true><<<stream_grid(n / Pack<T>::V), 256, 0, stream()>>>(n, key, prob, scaling_factor, x, y);
	else
		dropout_kernel<T, false><<<stream_grid(n), 256, 0, stream()>>>(n, key, prob, scaling_factor, x, y);
	check_launch();
}

/* ---- BroadcastLayer (layer/BroadcastLayer.hpp:69-101) --------------------------------------------
 * forward: out(n, h, w, c) = in(n, h mod H, w mod W, c mod C) on an output of (H bh, W bw, C bc);
 * backward: the replicas summed rank by rank as the reference does (first rank first, each sum from zero, slices in
 * order). The sample index is the contiguous one in both tensors. */
namespace {

struct BroadcastShape {
	int H, W, C, bh, bw, bc;
};

/* Both kernels use the pooling kernels' launch shape: a block covers a range of samples (VN per thread, 16-byte
 * accesses) and of rows of one (column, channel) pair of the input, so that the divisions run once per block. */
template<typename T, int VN>
__global__ __launch_bounds__(256)
void broadcast_forward_kernel(BroadcastShape s, int N, PoolLaunch pl, const T* __restrict__ x, T* __restrict__ out) {
	const size_t OH = (size_t) s.H * s.bh, OW = (size_t) s.W * s.bw;
	unsigned b = blockIdx.x;
	const int nb = (int) (b % (unsigned) pl.nblks);
	b /= (unsigned) pl.nblks;
	const int rb = (int) (b % (unsigned) pl.rblks);
	b /= (unsigned) pl.rblks;
	const int w = (int) (b % (unsigned) s.W);
	const int c = (int) (b / (unsigned) s.W);
	const int n = (nb * pl.tx + (int) threadIdx.x % pl.tx) * VN;
	if (n >= N)
		return;
	const int row0 = rb * pl.ty * POOL_ROWS + (int) threadIdx.x / pl.tx;
	#pragma unroll
	for (int j = 0; j < POOL_ROWS; ++j) {
		const int h = row0 + j * pl.ty;
		if (h >= s.H)
			break;
		/* an input element is read once and written to all its replicas */
		T v[VN];
		pool_load<T, VN>(v, x + n + (size_t) N * ((size_t) h + (size_t) s.H * ((size_t) w + (size_t) s.W * c)));
		for (int jc = 0; jc < s.bc; ++jc)
			for (int jw = 0; jw < s.bw; ++jw)
				for (int jh = 0; jh < s.bh; ++jh)
					pool_store<T, VN>(out + n + (size_t) N * (((size_t) h + (size_t) jh * s.H) +
							OH * (((size_t) w + (size_t) jw * s.W) + OW * ((size_t) c + (size_t) jc * s.C))), v);
	}
}

template<typename T, int VN>
__global__ __launch_bounds__(256)
void broadcast_backward_kernel(BroadcastShape s, int N, PoolLaunch pl, const T* __restrict__ g, T* __restrict__ dx) {
	const size_t OH = (size_t) s.H * s.bh, OW = (size_t) s.W * s.bw;
	unsigned b = blockIdx.x;
	const int nb = (int) (b % (unsigned) pl.nblks);
	b /= (unsigned) pl.nblks;
	const int rb = (int) (b % (unsigned) pl.rblks);
	b /= (unsigned) pl.rblks;
	const int w = (int) (b % (unsigned) s.W);
	const int c = (int) (b / (unsigned) s.W);
	const int n = (nb * pl.tx + (int) threadIdx.x % pl.tx) * VN;
	if (n >= N)
		return;
	const int row0 = rb * pl.ty * POOL_ROWS + (int) threadIdx.x / pl.tx;
	#pragma unroll
	for (int j = 0; j < POOL_ROWS; ++j) {
		const int h = row0 + j * pl.ty;
		if (h >= s.H)
			break;
		/* a rank that is not repeated is not summed over (no "0 +" for it): BroadcastLayer.hpp:86-87 */
		T sum_c[VN];
		for (int jc = 0; jc < s.bc; ++jc) {
			T sum_w[VN];
			for (int jw = 0; jw < s.bw; ++jw) {
				T sum_h[VN];
				for (int jh = 0; jh < s.bh; ++jh) {
					T e[VN];
					pool_load<T, VN>(e, g + n + (size_t) N * (((size_t) h + (size_t) jh * s.H) +
							OH * (((size_t) w + (size_t) jw * s.W) + OW * ((size_t) c + (size_t) jc * s.C))));
					#pragma unroll
					for (int v = 0; v < VN; ++v)
						sum_h[v] = jh == 0 ? (s.bh > 1 ? (T) 0 + e[v] : e[v]) : sum_h[v] + e[v];
				}
				#pragma unroll
				for (int v = 0; v < VN; ++v)
					sum_w[v] = jw == 0 ? (s.bw > 1 ? (T) 0 + sum_h[v] : sum_h[v]) : sum_w[v] + sum_h[v];
			}
			#pragma unroll
			for (int v = 0; v < VN; ++v)
				sum_c[v] = jc == 0 ? (s.bc > 1 ? (T) 0 + sum_w[v] : sum_w[v]) : sum_c[v] + sum_w[v];
		}
		pool_store<T, VN>(dx + n + (size_t) N * ((size_t) h + (size_t) s.H * ((size_t) w + (size_t) s.W * c)), sum_c);
	}
}

} /* namespace */

template<typename T>
void broadcast_forward(int H, int W, int C, int bh, int bw, int bc, int N, const T* x, T* out) {
	const BroadcastShape s = { H, W, C, bh, bw, bc };
	constexpr int VN = 16 / (int) sizeof(T);
	if (N % VN == 0 && aligned16(x) && aligned16(out)) {
		const PoolLaunch pl = pool_launch(N, H, VN);
		broadcast_forward_kernel<T, VN><<<pool_grid(pl, W, C), 256, 0, stream()>>>(s, N, pl, x, out);
	} else {
		const PoolLaunch pl = pool_launch(N, H, 1);
		broadcast_forward_kernel<T, 1><<<pool_grid(pl, W, C), 256, 0, stream()>>>(s, N, pl, x, out);
	}
	check_launch();
}

template<typename T>
void broadcast_backward(int H, int W, int C, int bh, int bw, int bc, int N, const T* out_grad, T* in_grad) {
	const BroadcastShape s = { H, W, C, bh, bw, bc };
	constexpr int VN = 16 / (int) sizeof(T);
	if (N % VN == 0 && aligned16(out_grad) && aligned16(in_grad)) {
		const PoolLaunch pl = pool_launch(N, H, VN);
		broadcast_backward_kernel<T, VN><<<pool_grid(pl, W, C), 256, 0, stream()>>>(s, N, pl, out_grad, in_grad);
	} else {
		const PoolLaunch pl = pool_launch(N, H, 1);
		broadcast_backward_kernel<T, 1><<<pool_grid(pl, W, C), 256, 0, stream()>>>(s, N, pl, out_grad, in_grad);
	}
	check_launch();
}

/* ----------------------------------------------------------------------------------------------
 * The element-wise and pooling layers behind a kernel layer, run as one pass each way (a fused kernel layer:
 * convolution or dense -> [batch norm] -> [activation] -> [pool]). `z` is the kernel layer's output (N, H, W, C);
 * pooling windows tile it exactly (stride = receptor, H % prh == 0, W % prw == 0). A thread owns V consecutive
 * samples of one window. Channel c is the slab [c * N*H*W, (c+1) * N*H*W) of z and [c * Lp, (c+1) * Lp) of the
 * pooled tensor, Lp = N * (H/prh) * (W/prw).
 * -------------------------------------------------------------------------------------------- */
namespace {

enum { CHAIN_POOL_NONE = 0, CHAIN_POOL_MAX = 1, CHAIN_POOL_MEAN = 2 };

template<typename T, int V> struct ChainVec { typedef T type __attribute__((ext_vector_type(V))); typedef unsigned utype __attribute__((ext_vector_type(V))); };
template<typename T> struct ChainVec<T, 1> { typedef T type; typedef unsigned utype; };

template<typename T, int V>
__device__ __forceinline__ void chain_load(T (&dst)[V], const T* p) {
	if constexpr (V == 1) {
		dst[0] = *p;
	} else {
		typedef T vt __attribute__((ext_vector_type(V)));
		const vt v = *reinterpret_cast<const vt*>(p);
		#pragma unroll
		for (int i = 0; i < V; ++i)
			dst[i] = v[i];
	}
}

template<typename T, int V>
__device__ __forceinline__ void chain_store(T* p, const T (&src)[V]) {
	if constexpr (V == 1) {
		*p = src[0];
	} else {
		typedef T vt __attribute__((ext_vector_type(V)));
		vt v;
		#pragma unroll
		for (int i = 0; i < V; ++i)
			v[i] = src[i];
		*reinterpret_cast<vt*>(p) = v;
	}
}

/* dz of a kernel layer followed by an activation and, with POOL, max pooling, from what the fused forward pass kept:
 * the (coded) output `y` or, for activations whose derivative needs it, the pre-activation values `pre` (at the
 * arg-max positions when pooled), and the arg-max cache. One thread per window and V samples:
 * dz(position) = g * act'(.) at the arg-max position, 0 elsewhere (MaxPoolLayer.hpp:66-80 followed by the
 * activation's pass_back). */
template<typename T, int V, int POOL>
__global__ __launch_bounds__(256)
void chain_backward_kernel(ChainShape s, int N, size_t total, const T* __restrict__ g, const unsigned* __restrict__ inds,
		const T* __restrict__ y, const T* __restrict__ pre, T* __restrict__ dz) {
	const size_t i = ((size_t) blockIdx.x * 256 + threadIdx.x) * V;
	if (i >= total)
		return;
	const int OHp = s.H / s.prh, OWp = s.W / s.prw;
	const int n = (int) (i % (size_t) N);
	size_t t = i / (size_t) N;
	const int a_p = (int) (t % (size_t) OHp);
	t /= (size_t) OHp;
	const int b_p = (int) (t % (size_t) OWp), c = (int) (t / (size_t) OWp);
	T gv[V], yv[V], gb[V];
	unsigned iv[V];
	chain_load<T, V>(gv, g + i);
	if constexpr (POOL == CHAIN_POOL_MEAN) {
		/* every position of the window receives g / (window size) (MeanPoolLayer.hpp:42-47) times the activation's
		 * derivative there: y / pre are full-size tensors */
		#pragma unroll
		for (int v = 0; v < V; ++v)
			gv[v] = gv[v] / (T) (s.prh * s.prw);
		const size_t first = n + (size_t) N * ((size_t) a_p * s.prh + (size_t) s.H * ((size_t) b_p * s.prw + (size_t) s.W * c));
		act_dispatch(s.kind, [&](auto kc) {
			constexpr int KIND = decltype(kc)::value;
			for (int k = 0; k < s.prw; ++k)
				for (int l = 0; l < s.prh; ++l) {
					const size_t at = first + (size_t) N * (l + (size_t) s.H * k);
					if (pre)
						chain_load<T, V>(yv, pre + at);
					else if (y)
						chain_load<T, V>(yv, y + at);
					#pragma unroll
					for (int v = 0; v < V; ++v)
						gb[v] = pre ? act_b<T, KIND>(yv[v], act_needs_y(KIND) ? act_f<T, KIND>(yv[v], (T) s.p) : (T) 0, gv[v], (T) s.p) :
								act_b_coded<T, KIND>(y ? yv[v] : (T) 0, gv[v], (T) s.p);
					chain_store<T, V>(dz + at, gb);
				}
		});
		return;
	}
	if (pre)
		chain_load<T, V>(yv, pre + i);
	else
		chain_load<T, V>(yv, y + i);
	act_dispatch(s.kind, [&](auto kc) {
		constexpr int KIND = decltype(kc)::value;
		#pragma unroll
		for (int v = 0; v < V; ++v)
			gb[v] = pre ? act_b<T, KIND>(yv[v], act_needs_y(KIND) ? act_f<T, KIND>(yv[v], (T) s.p) : (T) 0, gv[v], (T) s.p) :
					act_b_coded<T, KIND>(yv[v], gv[v], (T) s.p);
	});
	if constexpr (POOL == CHAIN_POOL_NONE) {
		chain_store<T, V>(dz + i, gb);
	} else {
		chain_load<unsigned, V>(iv, inds + (((size_t) b_p * OHp + a_p) * ((size_t) s.C * N) + (size_t) c * N + n));
		T* base = dz + n + (size_t) N * ((size_t) a_p * s.prh + (size_t) s.H * ((size_t) b_p * s.prw + (size_t) s.W * c));
		for (int k = 0; k < s.prw; ++k)
			for (int l = 0; l < s.prh; ++l) {
				T o[V];
				#pragma unroll
				for (int v = 0; v < V; ++v)
					o[v] = iv[v] == (unsigned) (k * s.prh + l) ? gb[v] : (T) 0;
				chain_store<T, V>(base + (size_t) N * (l + (size_t) s.H * k), o);
			}
	}
}

/* Per-channel moments of z from the per-tile moments the GEMM epilogue wrote (stats [mtiles][C][3]: count, mean,
 * sum of squared deviations): thread t merges tiles t, t + 256, ... in ascending order, then a fixed tree. */
template<typename T>
__device__ __forceinline__ void merge_tile_moments(const T* __restrict__ stats, int mtiles, int C, int c, T (*lds)[256], T& mean,
		T& m2) {
	const int tid = threadIdx.x;
	T n = (T) 0;
	mean = (T) 0;
	m2 = (T) 0;
	for (int tile = tid; tile < mtiles; tile += 256) {
		const T* e = stats + ((size_t) tile * C + c) * 3;
		moments_merge(n, mean, m2, e[0], e[1], e[2]);
	}
	lds[0][tid] = n;
	lds[1][tid] = mean;
	lds[2][tid] = m2;
	__syncthreads();
	for (int off = 128; off > 0; off >>= 1) {
		if (tid < off) {
			T a_n = lds[0][tid], a_mean = lds[1][tid], a_m2 = lds[2][tid];
			moments_merge(a_n, a_mean, a_m2, lds[0][tid + off], lds[1][tid + off], lds[2][tid + off]);
			lds[0][tid] = a_n;
			lds[1][tid] = a_mean;
			lds[2][tid] = a_m2;
		}
		__syncthreads();
	}
	mean = lds[1][0];
	m2 = lds[2][0];
}

/* (sample, pooled row, pooled column) of element i of a channel's pooled slab, kept up to date as i advances by a fixed
 * step: the divisions happen once per thread, each step costs two additions with carry (64-bit divisions per iteration
 * were most of the instructions of these loops). */
struct PooledWalk {
	int n, a, b;            /* i = n + N * (a + OHp * b) */
	int dn, da, db;         /* the step, decomposed the same way */
};
__device__ __forceinline__ PooledWalk pooled_walk(size_t i, unsigned step, int N, int OHp) {
	PooledWalk w;
	const unsigned i32 = (unsigned) i;      /* a slab has fewer than 2^31 elements */
	w.n = (int) (i32 % (unsigned) N);
	const unsigned t = i32 / (unsigned) N;
	w.a = (int) (t % (unsigned) OHp);
	w.b = (int) (t / (unsigned) OHp);
	w.dn = (int) (step % (unsigned) N);
	const unsigned dt = step / (unsigned) N;
	w.da = (int) (dt % (unsigned) OHp);
	w.db = (int) (dt / (unsigned) OHp);
	return w;
}
__device__ __forceinline__ void pooled_walk_next(PooledWalk& w, int N, int OHp) {
	w.n += w.dn;
	const int c1 = w.n >= N;
	w.n -= c1 ? N : 0;
	w.a += w.da + c1;
	const int c2 = w.a >= OHp;
	w.a -= c2 ? OHp : 0;
	w.b += w.db + c2;
}

struct ChainBn {
	int mtiles;             /* rows of the per-tile moments (training) */
	int training, stats_init;
	int merged;             /* training: mean_cache and inv_sd_cache already hold the batch moments (bn_merge_moments_kernel) */
};

/* Mean and inverse standard deviation of every channel from the per-tile moments, and the running averages' update
 * (BatchNormLayer.hpp:229-243), one block per channel: for launches with so many tiles that merging them in every block
 * of bn_chain_forward_kernel (a chain of dependent loads per thread, repeated by all blocks of a channel) would take
 * longer than a launch of its own. */
template<typename T>
__global__ __launch_bounds__(256)
void bn_merge_moments_kernel(const T* __restrict__ stats, int mtiles, int C, size_t L, T* __restrict__ avg_mean,
		T* __restrict__ avg_inv_sd, int stats_init, T decay, T eps, T* __restrict__ mean_cache, T* __restrict__ inv_sd_cache) {
	__shared__ T lds[3][256];
	const int c = blockIdx.x;
	T mean, m2;
	merge_tile_moments<T>(stats, mtiles, C, c, lds, mean, m2);
	if (threadIdx.x == 0) {
		const T inv_sd = (T) 1 / dev_sqrt(m2 / (T) L + eps);
		mean_cache[c] = mean;
		inv_sd_cache[c] = inv_sd;
		if (stats_init) {
			avg_mean[c] = ((T) 1 - decay) * avg_mean[c] + decay * mean;
			avg_inv_sd[c] = ((T) 1 - decay) * avg_inv_sd[c] + decay * inv_sd;
		} else {
			avg_mean[c] = mean;
			avg_inv_sd[c] = inv_sd;
		}
	}
}

/* Forward pass behind the kernel layer with batch norm: channel moments (training: merged from the tiles' moments;
 * inference: the running statistics), then y = act(gamma * (z - mean) * inv_sd + beta), pooled when POOL. The
 * backward pass recomputes what it needs from z, so only mean and inverse standard deviation are kept per channel
 * (BatchNormLayer.hpp:225-249 followed by the activation's and the pool's pass_forward). grid = (C, splits). */
template<typename T, int V, int POOL>
__global__ __launch_bounds__(256)
void bn_chain_forward_kernel(ChainShape s, int N, size_t span, ChainBn bn, const T* __restrict__ z, const T* __restrict__ stats,
		const T* __restrict__ gamma, const T* __restrict__ beta, T* __restrict__ avg_mean, T* __restrict__ avg_inv_sd, T decay, T eps,
		T* __restrict__ mean_cache, T* __restrict__ inv_sd_cache, T* __restrict__ out, unsigned* __restrict__ inds) {
	__shared__ T lds[3][256];
	const int c = blockIdx.x;
	const int OHp = s.H / s.prh, OWp = s.W / s.prw;
	const size_t L = (size_t) N * s.H * s.W, Lp = (size_t) N * OHp * OWp;
	T mean, inv_sd;
	if (bn.training && bn.merged) {
		mean = mean_cache[c];
		inv_sd = inv_sd_cache[c];
	} else if (bn.training) {
		T m2;
		merge_tile_moments<T>(stats, bn.mtiles, s.C, c, lds, mean, m2);
		inv_sd = (T) 1 / dev_sqrt(m2 / (T) L + eps);
		if (blockIdx.y == 0 && threadIdx.x == 0) {
			mean_cache[c] = mean;
			inv_sd_cache[c] = inv_sd;
			if (bn.stats_init) {       /* running average (BatchNormLayer.hpp:234-238) */
				avg_mean[c] = ((T) 1 - decay) * avg_mean[c] + decay * mean;
				avg_inv_sd[c] = ((T) 1 - decay) * avg_inv_sd[c] + decay * inv_sd;
			} else {                   /* first call assigns (:239-243) */
				avg_mean[c] = mean;
				avg_inv_sd[c] = inv_sd;
			}
		}
	} else {
		mean = avg_mean[c];
		inv_sd = avg_inv_sd[c];
	}
	const T ga = gamma[c], be = beta[c];
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < Lp ? begin + span : Lp;
	const T* zc = z + (size_t) c * L;
	T* oc = out + (size_t) c * Lp;
	act_dispatch(s.kind, [&](auto kc) {
		constexpr int KIND = decltype(kc)::value;
		PooledWalk walk = pooled_walk(begin + (size_t) threadIdx.x * V, 256u * V, N, OHp);
		for (size_t i = begin + (size_t) threadIdx.x * V; i < end; i += (size_t) 256 * V, pooled_walk_next(walk, N, OHp)) {
			const int n = walk.n, a_p = walk.a, b_p = walk.b;
			const T* base = zc + n + (size_t) N * ((size_t) a_p * s.prh + (size_t) s.H * ((size_t) b_p * s.prw));
			T res[V];
			unsigned bi[V];
			#pragma unroll
			for (int v = 0; v < V; ++v) {
				res[v] = POOL == CHAIN_POOL_MAX ? std::numeric_limits<T>::lowest() : (T) 0;
				bi[v] = 0;
			}
			for (int k = 0; k < s.prw; ++k)
				for (int l = 0; l < s.prh; ++l) {
					T zv[V];
					chain_load<T, V>(zv, base + (size_t) N * (l + (size_t) s.H * k));
					#pragma unroll
					for (int v = 0; v < V; ++v) {
						const T yv = act_f<T, KIND>(((zv[v] - mean) * inv_sd) * ga + be, (T) s.p);
						if (POOL == CHAIN_POOL_MAX) {
							if (yv > res[v]) {
								res[v] = yv;
								bi[v] = (unsigned) (k * s.prh + l);
							}
						} else {
							res[v] += yv;
						}
					}
				}
			if (POOL == CHAIN_POOL_MEAN) {
				#pragma unroll
				for (int v = 0; v < V; ++v)
					res[v] = res[v] / (T) (s.prh * s.prw);
			}
			chain_store<T, V>(oc + i, res);
			if (POOL == CHAIN_POOL_MAX)
				chain_store<unsigned, V>(inds + (((size_t) b_p * OHp + a_p) * ((size_t) s.C * N) + (size_t) c * N + n), bi);
		}
	});
}

/* The gradient that reaches the batch norm's output at the window positions of one pooled element, and the
 * normalised inputs there: g_bn = pool'(g) * act'(y_bn), recomputed from z. Calls fn(k, l, z, std, g_bn) per position
 * (max pooling: the arg-max position only when ONLY_NONZERO). */
template<typename T, int V, int POOL, int KIND, bool ONLY_NONZERO, typename Fn>
__device__ __forceinline__ void chain_bn_window(const ChainShape& s, int N, const T* base, const T (&gv)[V], const unsigned (&iv)[V],
		T mean, T inv_sd, T ga, T be, Fn fn) {
	const T area = (T) (s.prh * s.prw);
	if constexpr (POOL == CHAIN_POOL_MAX && ONLY_NONZERO) {
		#pragma unroll
		for (int v = 0; v < V; ++v) {
			const int k = (int) iv[v] / s.prh, l = (int) iv[v] - k * s.prh;
			const T zv = base[v + (size_t) N * (l + (size_t) s.H * k)];
			const T sd = (zv - mean) * inv_sd, yb = sd * ga + be;
			const T gb = act_b<T, KIND>(yb, act_needs_y(KIND) ? act_f<T, KIND>(yb, (T) s.p) : (T) 0, gv[v], (T) s.p);
			fn(v, sd, gb);
		}
	} else
	for (int k = 0; k < s.prw; ++k)
		for (int l = 0; l < s.prh; ++l) {
			T zv[V];
			chain_load<T, V>(zv, base + (size_t) N * (l + (size_t) s.H * k));
			#pragma unroll
			for (int v = 0; v < V; ++v) {
				const T sd = (zv[v] - mean) * inv_sd, yb = sd * ga + be;
				T up = gv[v];
				if (POOL == CHAIN_POOL_MEAN)
					up = up / area;
				T gb = act_b<T, KIND>(yb, act_needs_y(KIND) ? act_f<T, KIND>(yb, (T) s.p) : (T) 0, up, (T) s.p);
				if (POOL == CHAIN_POOL_MAX && iv[v] != (unsigned) (k * s.prh + l))
					gb = (T) 0;
				fn(v, k, l, sd, gb);
			}
		}
}

/* Sums over a channel of g_bn and of g_bn * std (BatchNormLayer.hpp:252-254), per split. grid = (C, splits). */
template<typename T, int V, int POOL>
__global__ __launch_bounds__(256)
void bn_chain_sums_kernel(ChainShape s, int N, size_t span, const T* __restrict__ g, const unsigned* __restrict__ inds,
		const T* __restrict__ z, const T* __restrict__ gamma, const T* __restrict__ beta, const T* __restrict__ mean_cache,
		const T* __restrict__ inv_sd_cache, T* __restrict__ ws_g, T* __restrict__ ws_gs) {
	__shared__ T lds[4];
	const int c = blockIdx.x;
	const int OHp = s.H / s.prh, OWp = s.W / s.prw;
	const size_t L = (size_t) N * s.H * s.W, Lp = (size_t) N * OHp * OWp;
	const T mean = mean_cache[c], inv_sd = inv_sd_cache[c], ga = gamma[c], be = beta[c];
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < Lp ? begin + span : Lp;
	const T* zc = z + (size_t) c * L;
	const T* gc = g + (size_t) c * Lp;
	T s1 = (T) 0, s2 = (T) 0;
	act_dispatch(s.kind, [&](auto kc) {
		constexpr int KIND = decltype(kc)::value;
		PooledWalk walk = pooled_walk(begin + (size_t) threadIdx.x * V, 256u * V, N, OHp);
		for (size_t i = begin + (size_t) threadIdx.x * V; i < end; i += (size_t) 256 * V, pooled_walk_next(walk, N, OHp)) {
			const int n = walk.n, a_p = walk.a, b_p = walk.b;
			const T* base = zc + n + (size_t) N * ((size_t) a_p * s.prh + (size_t) s.H * ((size_t) b_p * s.prw));
			T gv[V];
			unsigned iv[V];
			chain_load<T, V>(gv, gc + i);
			if (POOL == CHAIN_POOL_MAX)
				chain_load<unsigned, V>(iv, inds + (((size_t) b_p * OHp + a_p) * ((size_t) s.C * N) + (size_t) c * N + n));
			if constexpr (POOL == CHAIN_POOL_MAX)
				chain_bn_window<T, V, POOL, KIND, true>(s, N, base, gv, iv, mean, inv_sd, ga, be, [&](int, T sd, T gb) {
					s1 += gb;
					s2 += gb * sd;
				});
			else
				chain_bn_window<T, V, POOL, KIND, false>(s, N, base, gv, iv, mean, inv_sd, ga, be, [&](int, int, int, T sd, T gb) {
					s1 += gb;
					s2 += gb * sd;
				});
		}
	});
	s1 = block_sum_256(s1, lds);
	s2 = block_sum_256(s2, lds);
	if (threadIdx.x == 0) {
		ws_g[(size_t) c * gridDim.y + blockIdx.y] = s1;
		ws_gs[(size_t) c * gridDim.y + blockIdx.y] = s2;
	}
}

/* dz = (L * g_bn * gamma - sum(g_bn * gamma) - std * sum(std * g_bn * gamma)) * inv_sd / L at every position
 * (BatchNormLayer.hpp:257-261), gamma and beta gradients accumulated by the first split's first thread. */
template<typename T, int V, int POOL>
__global__ __launch_bounds__(256)
void bn_chain_apply_kernel(ChainShape s, int N, size_t span, const T* __restrict__ g, const unsigned* __restrict__ inds,
		const T* __restrict__ z, const T* __restrict__ gamma, const T* __restrict__ beta, const T* __restrict__ mean_cache,
		const T* __restrict__ inv_sd_cache, const T* __restrict__ ws_g, const T* __restrict__ ws_gs, T* __restrict__ gamma_grad,
		T* __restrict__ beta_grad, T* __restrict__ dz) {
	const int c = blockIdx.x, splits = gridDim.y;
	const int OHp = s.H / s.prh, OWp = s.W / s.prw;
	const size_t L = (size_t) N * s.H * s.W, Lp = (size_t) N * OHp * OWp;
	const T sum_g = sum_partials(ws_g + (size_t) c * splits, splits);
	const T sum_gs = sum_partials(ws_gs + (size_t) c * splits, splits);
	if (blockIdx.y == 0 && threadIdx.x == 0) {
		gamma_grad[c] += sum_gs;
		beta_grad[c] += sum_g;
	}
	const T mean = mean_cache[c], inv_sd = inv_sd_cache[c], ga = gamma[c], be = beta[c];
	const T sum_sg = sum_g * ga, sum_ssg = sum_gs * ga, scale = ((T) 1 / (T) L) * inv_sd;
	const size_t begin = (size_t) blockIdx.y * span, end = begin + span < Lp ? begin + span : Lp;
	const T* zc = z + (size_t) c * L;
	const T* gc = g + (size_t) c * Lp;
	T* dc = dz + (size_t) c * L;
	act_dispatch(s.kind, [&](auto kc) {
		constexpr int KIND = decltype(kc)::value;
		PooledWalk walk = pooled_walk(begin + (size_t) threadIdx.x * V, 256u * V, N, OHp);
		for (size_t i = begin + (size_t) threadIdx.x * V; i < end; i += (size_t) 256 * V, pooled_walk_next(walk, N, OHp)) {
			const int n = walk.n, a_p = walk.a, b_p = walk.b;
			const size_t off = n + (size_t) N * ((size_t) a_p * s.prh + (size_t) s.H * ((size_t) b_p * s.prw));
			T gv[V];
			unsigned iv[V];
			chain_load<T, V>(gv, gc + i);
			if (POOL == CHAIN_POOL_MAX)
				chain_load<unsigned, V>(iv, inds + (((size_t) b_p * OHp + a_p) * ((size_t) s.C * N) + (size_t) c * N + n));
			T o[V];
			chain_bn_window<T, V, POOL, KIND, false>(s, N, zc + off, gv, iv, mean, inv_sd, ga, be, [&](int v, int k, int l, T sd, T gb) {
				o[v] = (((T) L * (gb * ga) - sum_sg) - sd * sum_ssg) * scale;
				if (v == V - 1)
					chain_store<T, V>(dc + off + (size_t) N * (l + (size_t) s.H * k), o);
			});
		}
	});
}

unsigned chain_grid(size_t items) {
	const size_t blocks = (items + 255) / 256;
	CATTLE_HIP_REQUIRE(blocks < 2147483647u, "launch exceeds the grid limit");
	return (unsigned) std::max<size_t>(1, blocks);
}

template<typename T>
bool chain_vectors(int N, std::initializer_list<const void*> ptrs) {
	if (N % Pack<T>::V != 0)
		return false;
	for (const void* p : ptrs)
		if (p && !aligned16(p))
			return false;
	return true;
}

} /* namespace */

template<typename T>
void chain_backward(const ChainShape& s, int N, const T* g, const unsigned* inds, const T* y, const T* pre, T* dz) {
	const size_t total = (size_t) N * (s.H / s.prh) * (s.W / s.prw) * s.C;
	constexpr int V = Pack<T>::V;
	const bool vec = chain_vectors<T>(N, { g, inds, y, pre, dz });
	if (s.pool == CHAIN_POOL_MAX) {
		if (vec)
			chain_backward_kernel<T, V, CHAIN_POOL_MAX><<<chain_grid(total / V), 256, 0, stream()>>>(s, N, total, g, inds, y, pre, dz);
		else
			chain_backward_kernel<T, 1, CHAIN_POOL_MAX><<<chain_grid(total), 256, 0, stream()>>>(s, N, total, g, inds, y, pre, dz);
	} else if (s.pool == CHAIN_POOL_MEAN) {
		if (vec)
			chain_backward_kernel<T, V, CHAIN_POOL_MEAN><<<chain_grid(total / V), 256, 0, stream()>>>(s, N, total, g, inds, y, pre, dz);
		else
			chain_backward_kernel<T, 1, CHAIN_POOL_MEAN><<<chain_grid(total), 256, 0, stream()>>>(s, N, total, g, inds, y, pre, dz);
	} else {
		if (vec)
			chain_backward_kernel<T, V, CHAIN_POOL_NONE><<<chain_grid(total / V), 256, 0, stream()>>>(s, N, total, g, inds, y, pre, dz);
		else
			chain_backward_kernel<T, 1, CHAIN_POOL_NONE><<<chain_grid(total), 256, 0, stream()>>>(s, N, total, g, inds, y, pre, dz);
	}
	check_launch();
}

/* From this many tiles on the tiles' moments are merged by bn_merge_moments_kernel: measured on 256 x 56 x 56 x 64 (1568
 * tiles), merging inside bn_chain_forward_kernel took 26 of its 82 us; at 512 tiles it is two loads per thread. */
constexpr int BN_CHAIN_MERGE_TILES = 1024;

/* Splits of a channel's pooled positions over blocks in the fused chain kernels: a thread takes a vector of pooled
 * positions and their windows per turn, so spans of 1024 positions keep the 256 threads of a block busy for one turn
 * (128 x 8 x 8 pooled positions x 64 channels: 9.5 / 6.2 / 7.6 us with spans of 2048, about 2 us less in all with 1024). */
int bn_chain_splits(int channels, size_t Lp) {
	const size_t by_len = std::max<size_t>(1, Lp / 1024);
	const size_t by_fill = std::max<size_t>(1, (size_t) 2048 / (size_t) std::max(1, channels));
	return (int) std::min<size_t>(BN_MAX_SPLITS, std::min(by_len, by_fill));
}

size_t bn_chain_workspace(int channels) {
	return (size_t) 2 * channels * BN_MAX_SPLITS;
}

template<typename T, int V, int POOL>
void bn_chain_forward_launch(const ChainShape& s, int N, int mtiles, bool training, bool stats_init, const T* z, const T* stats,
		const T* gamma, const T* beta, T* avg_mean, T* avg_inv_sd, T decay, T eps, T* mean_cache, T* inv_sd_cache, T* out,
		unsigned* inds) {
	const size_t Lp = (size_t) N * (s.H / s.prh) * (s.W / s.prw);
	const int splits = bn_chain_splits(s.C, Lp);
	/* many tiles: their moments are merged once per channel by a launch of its own rather than by every block */
	const bool merged = training && mtiles >= BN_CHAIN_MERGE_TILES;
	if (merged) {
		bn_merge_moments_kernel<T><<<(unsigned) s.C, 256, 0, stream()>>>(stats, mtiles, s.C, (size_t) N * s.H * s.W, avg_mean, avg_inv_sd,
				stats_init ? 1 : 0, decay, eps, mean_cache, inv_sd_cache);
		check_launch();
	}
	const ChainBn bn = { mtiles, training ? 1 : 0, stats_init ? 1 : 0, merged ? 1 : 0 };
	bn_chain_forward_kernel<T, V, POOL><<<dim3((unsigned) s.C, (unsigned) splits), 256, 0, stream()>>>(s, N, bn_span(Lp, splits), bn, z,
			stats, gamma, beta, avg_mean, avg_inv_sd, decay, eps, mean_cache, inv_sd_cache, out, inds);
	check_launch();
}

template<typename T>
void bn_chain_forward(const ChainShape& s, int N, int mtiles, bool training, bool stats_init, const T* z, const T* stats,
		const T* gamma, const T* beta, T* avg_mean, T* avg_inv_sd, T decay, T eps, T* mean_cache, T* inv_sd_cache, T* out,
		unsigned* inds) {
	constexpr int V = Pack<T>::V;
	const bool vec = chain_vectors<T>(N, { z, out, inds });
	#define CATTLE_HIP_CHAIN_FWD(VV, PP) bn_chain_forward_launch<T, VV, PP>(s, N, mtiles, training, stats_init, z, stats, gamma, beta, \
			avg_mean, avg_inv_sd, decay, eps, mean_cache, inv_sd_cache, out, inds)
	if (s.pool == CHAIN_POOL_MAX) {
		if (vec) CATTLE_HIP_CHAIN_FWD(V, CHAIN_POOL_MAX); else CATTLE_HIP_CHAIN_FWD(1, CHAIN_POOL_MAX);
	} else if (s.pool == CHAIN_POOL_MEAN) {
		if (vec) CATTLE_HIP_CHAIN_FWD(V, CHAIN_POOL_MEAN); else CATTLE_HIP_CHAIN_FWD(1, CHAIN_POOL_MEAN);
	} else {
		if (vec) CATTLE_HIP_CHAIN_FWD(V, CHAIN_POOL_NONE); else CATTLE_HIP_CHAIN_FWD(1, CHAIN_POOL_NONE);
	}
	#undef CATTLE_HIP_CHAIN_FWD
}

template<typename T, int V, int POOL>
void bn_chain_backward_launch(const ChainShape& s, int N, const T* g, const unsigned* inds, const T* z, const T* gamma, const T* beta,
		const T* mean_cache, const T* inv_sd_cache, T* gamma_grad, T* beta_grad, T* dz, T* ws) {
	const size_t Lp = (size_t) N * (s.H / s.prh) * (s.W / s.prw);
	const int splits = bn_chain_splits(s.C, Lp);
	const size_t span = bn_span(Lp, splits);
	const dim3 grid((unsigned) s.C, (unsigned) splits);
	T* ws_g = ws;
	T* ws_gs = ws + (size_t) s.C * BN_MAX_SPLITS;
	bn_chain_sums_kernel<T, V, POOL><<<grid, 256, 0, stream()>>>(s, N, span, g, inds, z, gamma, beta, mean_cache, inv_sd_cache, ws_g, ws_gs);
	check_launch();
	bn_chain_apply_kernel<T, V, POOL><<<grid, 256, 0, stream()>>>(s, N, span, g, inds, z, gamma, beta, mean_cache, inv_sd_cache, ws_g, ws_gs,
			gamma_grad, beta_grad, dz);
	check_launch();
}

template<typename T>
void bn_chain_backward(const ChainShape& s, int N, const T* g, const unsigned* inds, const T* z, const T* gamma, const T* beta,
		const T* mean_cache, const T* inv_sd_cache, T* gamma_grad, T* beta_grad, T* dz, T* ws) {
	constexpr int V = Pack<T>::V;
	const bool vec = chain_vectors<T>(N, { g, inds, z, dz });
	#define CATTLE_HIP_CHAIN_BWD(VV, PP) bn_chain_backward_launch<T, VV, PP>(s, N, g, inds, z, gamma, beta, mean_cache, inv_sd_cache, \
			gamma_grad, beta_grad, dz, ws)
	if (s.pool == CHAIN_POOL_MAX) {
		if (vec) CATTLE_HIP_CHAIN_BWD(V, CHAIN_POOL_MAX); else CATTLE_HIP_CHAIN_BWD(1, CHAIN_POOL_MAX);
	} else if (s.pool == CHAIN_POOL_MEAN) {
		if (vec) CATTLE_HIP_CHAIN_BWD(V, CHAIN_POOL_MEAN); else CATTLE_HIP_CHAIN_BWD(1, CHAIN_POOL_MEAN);
	} else {
		if (vec) CATTLE_HIP_CHAIN_BWD(V, CHAIN_POOL_NONE); else CATTLE_HIP_CHAIN_BWD(1, CHAIN_POOL_NONE);
	}
	#undef CATTLE_HIP_CHAIN_BWD
}

#define CATTLE_HIP_INSTANTIATE(T) \
template void act_forward<T>(int, size_t, T, const T*, T*); \
template void chain_backward<T>(const ChainShape&, int, const T*, const unsigned*, const T*, const T*, T*); \
template void bn_chain_forward<T>(const ChainShape&, int, int, bool, bool, const T*, const T*, const T*, const T*, T*, T*, T, T, T*, T*, T*, unsigned*); \
template void bn_chain_backward<T>(const ChainShape&, int, const T*, const unsigned*, const T*, const T*, const T*, const T*, const T*, T*, T*, T*, T*); \
template void act_backward<T>(int, size_t, T, const T*, const T*, const T*, T*); \
template void softmax_forward<T>(int, int, T, const T*, T*); \
template void softmax_backward<T>(int, int, const T*, const T*, T*); \
template void prelu_forward<T>(int, int, const T*, const T*, T*); \
template void prelu_backward<T>(int, int, const T*, const T*, const T*, T*, T*); \
template void pswish_forward<T>(int, int, const T*, const T*, T*); \
template void pswish_backward<T>(int, int, const T*, const T*, const T*, T*, T*); \
template void bn_forward<T>(int, size_t, const T*, const T*, const T*, T*, T*, bool, bool, T, T, T*, T*, T*, T*); \
template void bn_backward<T>(int, size_t, const T*, const T*, const T*, const T*, T*, T*, T*, T*); \
template void maxpool_forward<T>(const PoolShape&, int, const T*, T*, unsigned*); \
template void maxpool_backward<T>(const PoolShape&, int, const T*, const unsigned*, T*); \
template void meanpool_forward<T>(const PoolShape&, int, const T*, T*); \
template void meanpool_backward<T>(const PoolShape&, int, const T*, T*); \
template void axpy_one<T>(size_t, const T*, T*); \
template void transpose_matrix<T>(int, int, const T*, T*, bool); \
template void add_row_vector<T>(int, size_t, const T*, T*); \
template void accumulate_column_sums<T>(int, size_t, const T*, T*); \
template void dropout_apply<T>(size_t, unsigned long long, T, T, const T*, T*); \
template void broadcast_forward<T>(int, int, int, int, int, int, int, const T*, T*); \
template void broadcast_backward<T>(int, int, int, int, int, int, int, const T*, T*); \
template void lstm_gates_forward<T>(const LstmForwardStep<T>&, const T*); \
template void lstm_gates_backward<T>(const LstmBackwardStep<T>&, const T*);

CATTLE_HIP_INSTANTIATE(float)
CATTLE_HIP_INSTANTIATE(double)

} /* namespace cattle_hip */
