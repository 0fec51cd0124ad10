/*
 * cattle_oracle.cpp — CPU restatement of C-ATTL3's kernel-layer algorithms.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. It exists so that the HIP kernels can be checked
 * against the algorithm of the reference on identical inputs, and so that the benchmark can time
 * a CPU baseline next to the GPU. Nothing in the product path may link or call it.
 *
 * The reference (ViktorC/C-ATTL3) delegates its arithmetic to Eigen, which is an un-vendored git
 * submodule and is absent; the reference therefore cannot be compiled. Every function below is a
 * plain-loop restatement of one reference function and cites it (paths relative to the reference
 * root, C-ATTL3/...). Buffers use the reference's memory layout: column-major tensors whose
 * index order is (N,H,W,C), so the offset of (n,h,w,c) is n + N*(h + H*(w + W*c))
 * (core/EigenProxy.hpp:43-64); matrices are column-major as well.
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   conv/dense fwd+bwd  pinned: 7-loop definitional cross-correlation, torch float64 conv2d,
 *                       adjoint identities, delta/box kernels, index-ordering probes.
 *   batch norm          pinned: closed-form invariants + torch float64 batch_norm.
 *   activations         pinned: libm/numpy closed forms and derivative-at-zero conventions.
 *   max/mean pool       pinned: brute force incl. crafted ties, NaN/-inf windows, overlaps.
 *   transposed conv     pinned: torch float64 conv_transpose2d with autograd, the adjoint identity with
 *                       the (pinned) convolution, output-size formula on the reference's test geometries.
 *   losses              pinned: torch float64 cross_entropy / mse / l1 / binary_cross_entropy / nll / kl_div /
 *                       multi_margin_loss (epsilon 0) with autograd for the gradients, hand-worked rows at the
 *                       hinge thresholds and with the epsilons, central differences of each loss against its gradient.
 *   dropout             pinned: the splitmix64 stream against its published outputs, the uniforms by their moments and
 *                       bin counts, the mask rule on hand-worked values. The reference's own random stream (Eigen's)
 *                       cannot be restated: which elements are dropped is "parity unpinned", by construction.
 *   broadcast           pinned: numpy.tile forward, torch autograd of a tiled tensor and the adjoint identity backward.
 *   other optimizers    pinned: torch's SGD (momentum, Nesterov), Adagrad, RMSprop, Adadelta and Adamax where the
 *                       recurrences coincide; first-step closed forms and the running-maximum property for
 *                       Nadam and AMSGrad, whose reference formulas differ from torch's.
 *   regularization      pinned: torch's weight decay (L2), hand-worked values, central differences of the penalty.
 *   SGD / Adam updates  pinned: numpy restatement in float64, first-step closed form, and torch's Adam
 *                       in the limit where the two formulas coincide.
 * What stays unpinned is only the bit pattern of Eigen's own summation order and of its
 * vectorised exp/tanh/log, which the reference's tests do not pin either (they hold no golden
 * vectors: test/gradient_test.cpp, test/training_test.cpp).
 */
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>
#include <algorithm>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef long long i64;

namespace {

/* ---------------------------------------------------------------------------------------------
 * Dense column-major GEMMs. Eigen's product kernels are replaced by cache-blocked loops; the
 * row-block loop is OpenMP-parallel to mirror Eigen's OpenMP GEMM (Makefile:7, -fopenmp).
 * ------------------------------------------------------------------------------------------- */
const i64 ROW_BLOCK = 256;

/* C[M x F] = A[M x K] * B[K x F]  (+ bias[f] broadcast over rows if bias != nullptr) */
template<typename T>
void gemm_nn(i64 M, i64 K, i64 F, const T* A, const T* B, const T* bias, T* C) {
	#pragma omp parallel for schedule(static)
	for (i64 m0 = 0; m0 < M; m0 += ROW_BLOCK) {
		const i64 mb = std::min(ROW_BLOCK, M - m0);
		for (i64 f = 0; f < F; ++f) {
			T* c = C + m0 + M * f;
			const T b0 = bias ? bias[f] : (T) 0;
			for (i64 i = 0; i < mb; ++i)
				c[i] = 0;
			for (i64 k = 0; k < K; ++k) {
				const T w = B[k + K * f];
				const T* a = A + m0 + M * k;
				for (i64 i = 0; i < mb; ++i)
					c[i] += a[i] * w;
			}
			if (bias)
				for (i64 i = 0; i < mb; ++i)
					c[i] += b0;
		}
	}
}

/* C[K x F] += A^T[K x M] * G[M x F] */
template<typename T>
void gemm_tn_acc(i64 M, i64 K, i64 F, const T* A, const T* G, T* C) {
	std::vector<T> prod((size_t) (K * F), (T) 0);
	#pragma omp parallel for schedule(static)
	for (i64 k = 0; k < K; ++k) {
		for (i64 m0 = 0; m0 < M; m0 += ROW_BLOCK) {
			const i64 mb = std::min(ROW_BLOCK, M - m0);
			const T* a = A + m0 + M * k;
			for (i64 f = 0; f < F; ++f) {
				const T* g = G + m0 + M * f;
				T s = 0;
				for (i64 i = 0; i < mb; ++i)
					s += a[i] * g[i];
				prod[(size_t) (k + K * f)] += s;
			}
		}
	}
	for (i64 i = 0; i < K * F; ++i)
		C[i] += prod[(size_t) i];
}

/* D[M x K] = G[M x F] * W^T[F x K], W stored [K x F] */
template<typename T>
void gemm_nt(i64 M, i64 K, i64 F, const T* G, const T* W, T* D) {
	#pragma omp parallel for schedule(static)
	for (i64 m0 = 0; m0 < M; m0 += ROW_BLOCK) {
		const i64 mb = std::min(ROW_BLOCK, M - m0);
		for (i64 k = 0; k < K; ++k) {
			T* d = D + m0 + M * k;
			for (i64 i = 0; i < mb; ++i)
				d[i] = 0;
			for (i64 f = 0; f < F; ++f) {
				const T w = W[k + K * f];
				const T* g = G + m0 + M * f;
				for (i64 i = 0; i < mb; ++i)
					d[i] += g[i] * w;
			}
		}
	}
}

/* colsum: out[f] += sum_m G[m,f]  (Eigen colwise().sum()); pairwise to keep fp32 error small */
template<typename T>
T pairwise_sum(const T* v, i64 n) {
	if (n <= 64) {
		T s = 0;
		for (i64 i = 0; i < n; ++i)
			s += v[i];
		return s;
	}
	const i64 h = n / 2;
	return pairwise_sum(v, h) + pairwise_sum(v + h, n - h);
}

template<typename T>
void colsum_acc(i64 M, i64 F, const T* G, T* out) {
	for (i64 f = 0; f < F; ++f)
		out[f] += pairwise_sum(G + M * f, M);
}

struct ConvGeom {
	i64 N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh;
	i64 PH, PW, DRH, DRW, OH, OW, M, K;
	void derive() {
		PH = H + 2 * pv;                       /* layer/kernel/ConvKernelLayer.hpp:69 */
		PW = W + 2 * ph;                       /* :70 */
		DRH = RH + (RH - 1) * dv;              /* :71 (dilation 0 = dense receptor) */
		DRW = RW + (RW - 1) * dh;              /* :72 */
		OH = (H - RH - (RH - 1) * dv + 2 * pv) / sv + 1;   /* :194-197 */
		OW = (W - RW - (RW - 1) * dh + 2 * ph) / sh + 1;
		M = N * OH * OW;
		K = RH * RW * C;
	}
};

/* layer/kernel/ConvKernelLayer.hpp:117-118 — zero padding on the H and W ranks only. */
template<typename T>
void pad_input(const ConvGeom& g, const T* x, std::vector<T>& xp) {
	xp.assign((size_t) (g.N * g.PH * g.PW * g.C), (T) 0);
	for (i64 c = 0; c < g.C; ++c)
		for (i64 w = 0; w < g.W; ++w)
			for (i64 h = 0; h < g.H; ++h)
				std::memcpy(&xp[(size_t) (g.N * ((h + g.pv) + g.PH * ((w + g.ph) + g.PW * c)))],
						x + g.N * (h + g.H * (w + g.W * c)), sizeof(T) * (size_t) g.N);
}

/* layer/kernel/ConvKernelLayer.hpp:125-142 — the materialised patch matrix [M x K]; patches are
 * enumerated with the horizontal offset in the outer loop and the vertical one in the inner loop,
 * each patch contributes N consecutive rows, and a patch tensor (N,RH,RW,C) viewed as an
 * N x (RH*RW*C) matrix gives column index rh + RH*(rw + RW*c). */
template<typename T>
void im2col(const ConvGeom& g, const T* xp, T* cache) {
	i64 patch_ind = 0;
	for (i64 i = 0; i <= g.PW - g.DRW; i += g.sh) {
		for (i64 j = 0; j <= g.PH - g.DRH; j += g.sv) {
			for (i64 c = 0; c < g.C; ++c)
				for (i64 rw = 0; rw < g.RW; ++rw)
					for (i64 rh = 0; rh < g.RH; ++rh) {
						const i64 col = rh + g.RH * (rw + g.RW * c);
						const T* src = xp + g.N * ((j + rh * (g.dv + 1)) +
								g.PH * ((i + rw * (g.dh + 1)) + g.PW * c));
						std::memcpy(cache + patch_ind + g.M * col, src, sizeof(T) * (size_t) g.N);
					}
			patch_ind += g.N;
		}
	}
}

/* layer/kernel/ConvKernelLayer.hpp:115-148 */
template<typename T>
int conv_forward(ConvGeom g, const T* x, const T* w, const T* b, T* out, T* cache) {
	g.derive();
	std::vector<T> xp;
	const T* src = x;
	if (g.pv > 0 || g.ph > 0) {
		pad_input(g, x, xp);
		src = xp.data();
	}
	std::vector<T> own;
	if (!cache) {
		own.resize((size_t) (g.M * g.K));
		cache = own.data();
	}
	im2col(g, src, cache);
	gemm_nn(g.M, g.K, g.F, cache, w, b, out);                /* :144-145 */
	return 0;
}

/* layer/kernel/ConvKernelLayer.hpp:149-189. wgrad and bgrad accumulate (StandardParameters.hpp:119).
 * in_grad == nullptr reproduces the input-layer early-out (:156-157). */
template<typename T>
int conv_backward(ConvGeom g, const T* cache, const T* w, const T* out_grad, T* wgrad, T* bgrad, T* in_grad) {
	g.derive();
	gemm_tn_acc(g.M, g.K, g.F, cache, out_grad, wgrad);       /* :154 */
	colsum_acc(g.M, g.F, out_grad, bgrad);                    /* :155 */
	if (!in_grad)
		return 0;
	std::vector<T> D((size_t) (g.M * g.K));
	gemm_nt(g.M, g.K, g.F, out_grad, w, D.data());            /* :159 */
	std::vector<T> pg((size_t) (g.N * g.PH * g.PW * g.C), (T) 0);   /* :162-163 */
	i64 patch_ind = 0;
	for (i64 i = 0; i <= g.PW - g.DRW; i += g.sh) {           /* :166-181, col2im in the same patch order */
		for (i64 j = 0; j <= g.PH - g.DRH; j += g.sv) {
			for (i64 c = 0; c < g.C; ++c)
				for (i64 rw = 0; rw < g.RW; ++rw)
					for (i64 rh = 0; rh < g.RH; ++rh) {
						const i64 col = rh + g.RH * (rw + g.RW * c);
						T* dst = &pg[(size_t) (g.N * ((j + rh * (g.dv + 1)) +
								g.PH * ((i + rw * (g.dh + 1)) + g.PW * c)))];
						const T* s = &D[(size_t) (patch_ind + g.M * col)];
						for (i64 n = 0; n < g.N; ++n)
							dst[n] += s[n];
					}
			patch_ind += g.N;
		}
	}
	for (i64 c = 0; c < g.C; ++c)                               /* :183-188, crop the padding */
		for (i64 wv = 0; wv < g.W; ++wv)
			for (i64 h = 0; h < g.H; ++h)
				std::memcpy(in_grad + g.N * (h + g.H * (wv + g.W * c)),
						&pg[(size_t) (g.N * ((h + g.pv) + g.PH * ((wv + g.ph) + g.PW * c)))],
						sizeof(T) * (size_t) g.N);
	return 0;
}

/* layer/kernel/DenseKernelLayer.hpp:92-102 */
template<typename T>
int dense_forward(i64 N, i64 V, i64 O, const T* x, const T* w, const T* b, T* out) {
	gemm_nn(N, V, O, x, w, b, out);
	return 0;
}

/* layer/kernel/DenseKernelLayer.hpp:103-115 */
template<typename T>
int dense_backward(i64 N, i64 V, i64 O, const T* x, const T* w, const T* out_grad, T* wgrad, T* bgrad, T* in_grad) {
	gemm_tn_acc(N, V, O, x, out_grad, wgrad);                   /* :108 */
	colsum_acc(N, O, out_grad, bgrad);                          /* :109 */
	if (in_grad)
		gemm_nt(N, V, O, out_grad, w, in_grad);                 /* :113 */
	return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Batch normalisation.
 * groups = number of statistics groups, L = elements per group.
 *   per-channel (layer/BatchNormLayer.hpp:170-262): group i is the contiguous slab
 *     [i*L, (i+1)*L), L = N*H*W; params are per-channel scalars.
 *   per-activation (:411-456): group i is column i of the N x vol matrix, L = N; it is the same
 *     memory pattern (contiguous column), so one routine serves both.
 * stats_init != 0 means the running statistics already hold values (avgs_init, :234-243).
 * ------------------------------------------------------------------------------------------- */
template<typename T>
int bn_forward(i64 groups, i64 L, const T* x, const T* gamma, const T* beta, T* avg_mean, T* avg_inv_sd,
		int stats_init, int training, T decay, T eps, T* out, T* std_cache, T* inv_sd_cache) {
	std::vector<T> tmp((size_t) L);
	for (i64 gidx = 0; gidx < groups; ++gidx) {
		const T* xs = x + gidx * L;
		T* ys = out + gidx * L;
		if (training) {
			const T mean = pairwise_sum(xs, L) / (T) L;                       /* :229 */
			for (i64 i = 0; i < L; ++i) {
				const T d = xs[i] - mean;                                     /* :230 */
				tmp[(size_t) i] = d * d;
			}
			const T inv_sd = (T) 1 / std::sqrt(pairwise_sum(tmp.data(), L) / (T) L + eps);   /* :231 */
			inv_sd_cache[gidx] = inv_sd;
			T* sc = std_cache + gidx * L;
			for (i64 i = 0; i < L; ++i)
				sc[i] = (xs[i] - mean) * inv_sd;                              /* :232 */
			if (stats_init) {                                                 /* :234-238 */
				avg_mean[gidx] = ((T) 1 - decay) * avg_mean[gidx] + decay * mean;
				avg_inv_sd[gidx] = ((T) 1 - decay) * avg_inv_sd[gidx] + decay * inv_sd;
			} else {                                                          /* :239-243 */
				avg_mean[gidx] = mean;
				avg_inv_sd[gidx] = inv_sd;
			}
			for (i64 i = 0; i < L; ++i)
				ys[i] = sc[i] * gamma[gidx] + beta[gidx];                     /* :248 */
		} else {
			for (i64 i = 0; i < L; ++i)                                       /* :246, :248 */
				ys[i] = ((xs[i] - avg_mean[gidx]) * avg_inv_sd[gidx]) * gamma[gidx] + beta[gidx];
		}
	}
	return 0;
}

/* layer/BatchNormLayer.hpp:250-262 (per-channel) and :441-456 (per-activation). */
template<typename T>
int bn_backward(i64 groups, i64 L, const T* out_grad, const T* gamma, const T* std_cache, const T* inv_sd_cache,
		T* gamma_grad, T* beta_grad, T* in_grad) {
	std::vector<T> tmp((size_t) L);
	for (i64 gidx = 0; gidx < groups; ++gidx) {
		const T* g = out_grad + gidx * L;
		const T* sc = std_cache + gidx * L;
		for (i64 i = 0; i < L; ++i)
			tmp[(size_t) i] = g[i] * sc[i];
		gamma_grad[gidx] += pairwise_sum(tmp.data(), L);                      /* :252-253 */
		beta_grad[gidx] += pairwise_sum(g, L);                                /* :254 */
		if (!in_grad)
			continue;
		/* std_in_grad = g * gamma (:256); sums of it and of std_in * std_in_grad (:257-259) */
		for (i64 i = 0; i < L; ++i)
			tmp[(size_t) i] = g[i] * gamma[gidx];
		const T sum_sg = pairwise_sum(tmp.data(), L);
		std::vector<T> tmp2((size_t) L);
		for (i64 i = 0; i < L; ++i)
			tmp2[(size_t) i] = sc[i] * tmp[(size_t) i];
		const T sum_ssg = pairwise_sum(tmp2.data(), L);
		const T scale = ((T) 1 / (T) L) * inv_sd_cache[gidx];                 /* :260-261 */
		T* dx = in_grad + gidx * L;
		for (i64 i = 0; i < L; ++i)
			dx[i] = (((T) L * tmp[(size_t) i] - sum_sg) - sc[i] * sum_ssg) * scale;
	}
	return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Activations. kind codes are shared with the C-ABI of the HIP library.
 * fwd produces out and up to two caches exactly as the reference layers keep them.
 * ------------------------------------------------------------------------------------------- */
enum ActKind {
	ACT_IDENTITY = 0, ACT_SCALED = 1, ACT_BINARY_STEP = 2, ACT_SIGMOID = 3, ACT_TANH = 4, ACT_SOFTSIGN = 5,
	ACT_SOFTPLUS = 6, ACT_RELU = 7, ACT_LEAKY_RELU = 8, ACT_ELU = 9, ACT_SWISH = 10
};

template<typename T>
int act_forward(int kind, i64 n, T p, const T* x, T* y) {
	switch (kind) {
	case ACT_IDENTITY:      /* layer/activation/IdentityActivationLayer.hpp:37-42 */
		for (i64 i = 0; i < n; ++i) y[i] = x[i];
		break;
	case ACT_SCALED:        /* ScaledActivationLayer.hpp:38-43 */
		for (i64 i = 0; i < n; ++i) y[i] = x[i] * p;
		break;
	case ACT_BINARY_STEP:   /* BinaryStepActivationLayer.hpp:42-47 */
		for (i64 i = 0; i < n; ++i) y[i] = (T) (x[i] >= 0);
		break;
	case ACT_SIGMOID:       /* SigmoidActivationLayer.hpp:38-43 */
		for (i64 i = 0; i < n; ++i) y[i] = (T) 1 / (std::exp(-x[i]) + (T) 1);
		break;
	case ACT_TANH:          /* TanhActivationLayer.hpp:38-43 */
		for (i64 i = 0; i < n; ++i) y[i] = std::tanh(x[i]);
		break;
	case ACT_SOFTSIGN:      /* SoftsignActivationLayer.hpp:39-44 */
		for (i64 i = 0; i < n; ++i) y[i] = x[i] / ((T) 1 + std::abs(x[i]));
		break;
	case ACT_SOFTPLUS:      /* SoftplusActivationLayer.hpp:40-45 (no overflow guard in the reference) */
		for (i64 i = 0; i < n; ++i) y[i] = std::log(std::exp(x[i]) + (T) 1);
		break;
	case ACT_RELU:          /* ReLUActivationLayer.hpp:45-50 */
		for (i64 i = 0; i < n; ++i) y[i] = std::max(x[i], (T) 0);
		break;
	case ACT_LEAKY_RELU:    /* LeakyReLUActivationLayer.hpp:50-55: max(x, alpha*x) */
		for (i64 i = 0; i < n; ++i) y[i] = std::max(x[i], x[i] * p);
		break;
	case ACT_ELU:           /* ELUActivationLayer.hpp:55-64 */
		for (i64 i = 0; i < n; ++i) y[i] = x[i] >= 0 ? x[i] : p * (std::exp(x[i]) - (T) 1);
		break;
	case ACT_SWISH:         /* SwishActivationLayer.hpp:45-51 */
		for (i64 i = 0; i < n; ++i) y[i] = x[i] * ((T) 1 / (std::exp(-p * x[i]) + (T) 1));
		break;
	default:
		return 1;
	}
	return 0;
}

/* x = forward input, y = forward output (both are given; each kind reads what its reference
 * layer caches). */
template<typename T>
int act_backward(int kind, i64 n, T p, const T* x, const T* y, const T* g, T* dx) {
	switch (kind) {
	case ACT_IDENTITY:      /* IdentityActivationLayer.hpp:43-49 */
		for (i64 i = 0; i < n; ++i) dx[i] = g[i];
		break;
	case ACT_SCALED:        /* ScaledActivationLayer.hpp:44-50 */
		for (i64 i = 0; i < n; ++i) dx[i] = g[i] * p;
		break;
	case ACT_BINARY_STEP:   /* BinaryStepActivationLayer.hpp:48-54 */
		for (i64 i = 0; i < n; ++i) dx[i] = 0;
		break;
	case ACT_SIGMOID:       /* SigmoidActivationLayer.hpp:44-50 */
		for (i64 i = 0; i < n; ++i) dx[i] = (y[i] * ((T) 1 - y[i])) * g[i];
		break;
	case ACT_TANH:          /* TanhActivationLayer.hpp:44-50 */
		for (i64 i = 0; i < n; ++i) dx[i] = ((T) 1 - y[i] * y[i]) * g[i];
		break;
	case ACT_SOFTSIGN: {    /* SoftsignActivationLayer.hpp:45-51 */
		for (i64 i = 0; i < n; ++i) {
			const T d = (T) 1 + std::abs(x[i]);
			dx[i] = ((T) 1 / (d * d)) * g[i];
		}
		break;
	}
	case ACT_SOFTPLUS:      /* SoftplusActivationLayer.hpp:46-52 */
		for (i64 i = 0; i < n; ++i) dx[i] = ((T) 1 / (std::exp(-x[i]) + (T) 1)) * g[i];
		break;
	case ACT_RELU:          /* ReLUActivationLayer.hpp:51-57: derivative 1 at x == 0 */
		for (i64 i = 0; i < n; ++i) dx[i] = (T) (x[i] >= 0) * g[i];
		break;
	case ACT_LEAKY_RELU:    /* LeakyReLUActivationLayer.hpp:56-62 */
		for (i64 i = 0; i < n; ++i) dx[i] = (x[i] >= 0 ? (T) 1 : p) * g[i];
		break;
	case ACT_ELU:           /* ELUActivationLayer.hpp:65-78 */
		for (i64 i = 0; i < n; ++i) dx[i] = (x[i] >= 0 ? (T) 1 : (y[i] + p)) * g[i];
		break;
	case ACT_SWISH: {       /* SwishActivationLayer.hpp:52-59 */
		for (i64 i = 0; i < n; ++i) {
			const T s = (T) 1 / (std::exp(-p * x[i]) + (T) 1);
			dx[i] = s * ((((T) 1 - s) * p) * x[i] + (T) 1) * g[i];
		}
		break;
	}
	default:
		return 1;
	}
	return 0;
}

/* layer/activation/SoftmaxActivationLayer.hpp:49-62; rows = samples of the N x V matrix. */
template<typename T>
int softmax_forward(i64 N, i64 V, T eps, const T* x, T* y) {
	for (i64 n = 0; n < N; ++n) {
		T mx = x[n];
		for (i64 v = 1; v < V; ++v)
			mx = std::max(mx, x[n + N * v]);
		T s = 0;
		for (i64 v = 0; v < V; ++v) {
			const T e = std::exp(x[n + N * v] - mx);
			y[n + N * v] = e;
			s += e;
		}
		for (i64 v = 0; v < V; ++v)
			y[n + N * v] /= (s + eps);
	}
	return 0;
}

/* SoftmaxActivationLayer.hpp:63-78: dx_row = g_row * (diag(y) - y^T y) */
template<typename T>
int softmax_backward(i64 N, i64 V, const T* y, const T* g, T* dx) {
	for (i64 n = 0; n < N; ++n) {
		for (i64 j = 0; j < V; ++j) {
			T s = 0;
			for (i64 i = 0; i < V; ++i) {
				const T jac = (i == j ? y[n + N * i] : (T) 0) - y[n + N * i] * y[n + N * j];
				s += g[n + N * i] * jac;
			}
			dx[n + N * j] = s;
		}
	}
	return 0;
}

/* layer/activation/PReLUActivationLayer.hpp:80-109; alpha is a 1 x V row vector. */
template<typename T>
int prelu_forward(i64 N, i64 V, const T* alpha, const T* x, T* y) {
	for (i64 v = 0; v < V; ++v)
		for (i64 n = 0; n < N; ++n)
			y[n + N * v] = std::max(x[n + N * v], x[n + N * v] * alpha[v]);   /* :85 */
	return 0;
}

template<typename T>
int prelu_backward(i64 N, i64 V, const T* alpha, const T* x, const T* g, T* alpha_grad, T* dx) {
	for (i64 v = 0; v < V; ++v) {
		T ag = 0;
		for (i64 n = 0; n < N; ++n) {
			const T xi = x[n + N * v], gi = g[n + N * v];
			if (xi >= 0) {
				if (dx) dx[n + N * v] = gi;
			} else {
				if (dx) dx[n + N * v] = alpha[v] * gi;
				ag += xi * gi;                                                /* :102 */
			}
		}
		alpha_grad[v] += ag;
	}
	return 0;
}

/* layer/activation/PSwishActivationLayer.hpp:77-99; beta is a 1 x V row vector. */
template<typename T>
int pswish_forward(i64 N, i64 V, const T* beta, const T* x, T* y) {
	for (i64 v = 0; v < V; ++v)
		for (i64 n = 0; n < N; ++n) {
			const T xi = x[n + N * v];
			y[n + N * v] = xi * ((T) 1 / (std::exp(xi * (-beta[v])) + (T) 1));
		}
	return 0;
}

template<typename T>
int pswish_backward(i64 N, i64 V, const T* beta, const T* x, const T* g, T* beta_grad, T* dx) {
	std::vector<T> col((size_t) N);
	for (i64 v = 0; v < V; ++v) {
		for (i64 n = 0; n < N; ++n) {
			const T xi = x[n + N * v], gi = g[n + N * v];
			const T s = (T) 1 / (std::exp(xi * (-beta[v])) + (T) 1);
			col[(size_t) n] = s * ((T) 1 - s) * xi * xi * gi;                /* :90-91 */
			if (dx)
				dx[n + N * v] = s * ((((T) 1 - s) * beta[v]) * xi + (T) 1) * gi;   /* :94-96 */
		}
		beta_grad[v] += pairwise_sum(col.data(), N);
	}
	return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Pooling. layer/PoolLayer.hpp:77-116 drives windows with the horizontal offset outer and the
 * vertical one inner; there is no padding or dilation and windows that do not fit are dropped.
 * ------------------------------------------------------------------------------------------- */
struct PoolGeom {
	i64 N, H, W, C, RH, RW, sv, sh, OH, OW;
	void derive() {
		OH = (H - RH) / sv + 1;               /* layer/PoolLayer.hpp:145-148 */
		OW = (W - RW) / sh + 1;
	}
};

/* layer/pool/MaxPoolLayer.hpp:38-64. inds has OH*OW rows of C*N entries: inds[patch][c*N + n] with
 * patch = ow_idx*OH + oh_idx; value = w_in_window*RH + h_in_window. */
template<typename T>
int maxpool_forward(PoolGeom g, const T* x, T* out, unsigned* inds) {
	g.derive();
	i64 patch = 0;
	for (i64 ow = 0; ow < g.OW; ++ow)
		for (i64 oh = 0; oh < g.OH; ++oh, ++patch)
			for (i64 c = 0; c < g.C; ++c)
				for (i64 n = 0; n < g.N; ++n) {
					T mx = std::numeric_limits<T>::lowest();      /* core/NumericUtils.hpp:26 */
					unsigned mh = 0, mw = 0;
					for (i64 k = 0; k < g.RW; ++k)
						for (i64 l = 0; l < g.RH; ++l) {
							const T v = x[n + g.N * ((oh * g.sv + l) + g.H * ((ow * g.sh + k) + g.W * c))];
							if (v > mx) {
								mx = v;
								mh = (unsigned) l;
								mw = (unsigned) k;
							}
						}
					inds[patch * (g.C * g.N) + c * g.N + n] = mw * (unsigned) g.RH + mh;
					out[n + g.N * (oh + g.OH * (ow + g.OW * c))] = mx;
				}
	return 0;
}

/* layer/pool/MaxPoolLayer.hpp:65-80 + layer/PoolLayer.hpp:96-116 (accumulation over overlaps). */
template<typename T>
int maxpool_backward(PoolGeom g, const T* out_grad, const unsigned* inds, T* in_grad) {
	g.derive();
	std::fill(in_grad, in_grad + g.N * g.H * g.W * g.C, (T) 0);
	i64 patch = 0;
	for (i64 ow = 0; ow < g.OW; ++ow)
		for (i64 oh = 0; oh < g.OH; ++oh, ++patch)
			for (i64 c = 0; c < g.C; ++c)
				for (i64 n = 0; n < g.N; ++n) {
					const unsigned ind = inds[patch * (g.C * g.N) + c * g.N + n];
					const i64 mh = ind % (unsigned) g.RH, mw = ind / (unsigned) g.RH;
					in_grad[n + g.N * ((oh * g.sv + mh) + g.H * ((ow * g.sh + mw) + g.W * c))] +=
							out_grad[n + g.N * (oh + g.OH * (ow + g.OW * c))];
				}
	return 0;
}

/* layer/pool/MeanPoolLayer.hpp:35-38 */
template<typename T>
int meanpool_forward(PoolGeom g, const T* x, T* out) {
	g.derive();
	for (i64 c = 0; c < g.C; ++c)
		for (i64 ow = 0; ow < g.OW; ++ow)
			for (i64 oh = 0; oh < g.OH; ++oh)
				for (i64 n = 0; n < g.N; ++n) {
					T s = 0;
					for (i64 k = 0; k < g.RW; ++k)
						for (i64 l = 0; l < g.RH; ++l)
							s += x[n + g.N * ((oh * g.sv + l) + g.H * ((ow * g.sh + k) + g.W * c))];
					out[n + g.N * (oh + g.OH * (ow + g.OW * c))] = s / (T) (g.RH * g.RW);
				}
	return 0;
}

/* layer/pool/MeanPoolLayer.hpp:39-41 + layer/PoolLayer.hpp:96-116 */
template<typename T>
int meanpool_backward(PoolGeom g, const T* out_grad, T* in_grad) {
	g.derive();
	std::fill(in_grad, in_grad + g.N * g.H * g.W * g.C, (T) 0);
	const T area = (T) (g.RH * g.RW);
	for (i64 ow = 0; ow < g.OW; ++ow)
		for (i64 oh = 0; oh < g.OH; ++oh)
			for (i64 c = 0; c < g.C; ++c)
				for (i64 k = 0; k < g.RW; ++k)
					for (i64 l = 0; l < g.RH; ++l)
						for (i64 n = 0; n < g.N; ++n)
							in_grad[n + g.N * ((oh * g.sv + l) + g.H * ((ow * g.sh + k) + g.W * c))] +=
									out_grad[n + g.N * (oh + g.OH * (ow + g.OW * c))] / area;
	return 0;
}

/* ---------------------------------------------------------------------------------------------
 * TransConvKernelLayerBase::_pass_forward / _pass_back (layer/kernel/TransConvKernelLayer.hpp:143-216),
 * restated with the reference's own staging: in_mat[(n, ih, iw) x C] * W[C x RH*RW*F], each row's
 * receptor patch added into the zero-padded output (width-major / height-minor patch order, :153-169),
 * padding cut off, per-activation bias added; backward gathers the same patches from the padded output
 * gradient into a matrix and multiplies (:186-214).
 * ------------------------------------------------------------------------------------------- */
struct TransGeom {
	i64 N, IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh;
	i64 OH, OW, PH, PW, DRH, DRW;
	void derive() {
		DRH = RH + (RH - 1) * dv;
		DRW = RW + (RW - 1) * dh;
		OH = (IH - 1) * sv + DRH - 2 * pv;      /* calculate_spatial_output_dim :226-229 */
		OW = (IW - 1) * sh + DRW - 2 * ph;
		PH = OH + 2 * pv;
		PW = OW + 2 * ph;
	}
};

template<typename T>
int transconv_forward(TransGeom g, const T* x, const T* w, const T* bias, T* out) {
	g.derive();
	const i64 M = g.N * g.IH * g.IW, RV = g.RH * g.RW * g.F;
	std::vector<T> conv_mat((size_t) (M * RV));
	gemm_nn<T>(M, g.C, RV, x, w, nullptr, conv_mat.data());
	std::vector<T> padded((size_t) (g.N * g.PH * g.PW * g.F), (T) 0);
	i64 patch = 0;
	for (i64 i = 0; i + g.DRW <= g.PW; i += g.sh)
		for (i64 j = 0; j + g.DRH <= g.PH; j += g.sv) {
			for (i64 f = 0; f < g.F; ++f)
				for (i64 rw = 0; rw < g.RW; ++rw)
					for (i64 rh = 0; rh < g.RH; ++rh)
						for (i64 n = 0; n < g.N; ++n)
							padded[n + g.N * ((j + rh * (g.dv + 1)) + g.PH * ((i + rw * (g.dh + 1)) + g.PW * f))] +=
									conv_mat[(patch + n) + M * (rh + g.RH * (rw + g.RW * f))];
			patch += g.N;
		}
	if (patch != M)
		return 1;
	for (i64 f = 0; f < g.F; ++f)
		for (i64 ow = 0; ow < g.OW; ++ow)
			for (i64 oh = 0; oh < g.OH; ++oh)
				for (i64 n = 0; n < g.N; ++n)
					out[n + g.N * (oh + g.OH * (ow + g.OW * f))] =
							padded[n + g.N * ((oh + g.pv) + g.PH * ((ow + g.ph) + g.PW * f))] + bias[oh + g.OH * (ow + g.OW * f)];
	return 0;
}

template<typename T>
int transconv_backward(TransGeom g, const T* x, const T* w, const T* out_grad, T* wgrad, T* bgrad, T* in_grad) {
	g.derive();
	const i64 M = g.N * g.IH * g.IW, RV = g.RH * g.RW * g.F, OV = g.OH * g.OW * g.F;
	for (i64 e = 0; e < OV; ++e) {
		T s = 0;
		for (i64 n = 0; n < g.N; ++n)
			s += out_grad[n + g.N * e];
		bgrad[e] += s;
	}
	std::vector<T> patches((size_t) (M * RV));
	i64 patch = 0;
	for (i64 i = 0; i + g.DRW <= g.PW; i += g.sh)
		for (i64 j = 0; j + g.DRH <= g.PH; j += g.sv) {
			for (i64 f = 0; f < g.F; ++f)
				for (i64 rw = 0; rw < g.RW; ++rw)
					for (i64 rh = 0; rh < g.RH; ++rh) {
						const i64 oh = j + rh * (g.dv + 1) - g.pv, ow = i + rw * (g.dh + 1) - g.ph;
						const bool inside = oh >= 0 && oh < g.OH && ow >= 0 && ow < g.OW;
						for (i64 n = 0; n < g.N; ++n)
							patches[(patch + n) + M * (rh + g.RH * (rw + g.RW * f))] =
									inside ? out_grad[n + g.N * (oh + g.OH * (ow + g.OW * f))] : (T) 0;
					}
			patch += g.N;
		}
	if (patch != M)
		return 1;
	gemm_tn_acc<T>(M, g.C, RV, x, patches.data(), wgrad);          /* in_mat_cache^T * out_grad_conv_mat (:208) */
	if (in_grad)
		gemm_nt<T>(M, g.C, RV, patches.data(), w, in_grad);        /* out_grad_conv_mat * W^T (:211) */
	return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Losses under the UniversalLoss drivers (loss/UniversalLoss.hpp:37-46 non-sequential; :99-125
 * sequential: every time step is sliced out and treated as its own rows x cols matrix, losses add up
 * over the steps). A batch is (N, T, V) column-major; T = 1 is the non-sequential case.
 *   0  loss/SquaredLoss.hpp:25-34               1  loss/SoftmaxCrossEntropyLoss.hpp:33-50
 *   2  loss/AbsoluteLoss.hpp:25-35              3  loss/BinaryCrossEntropyLoss.hpp:35-46 (V must be 1)
 *   4  loss/CrossEntropyLoss.hpp:33-42          5  loss/KullbackLeiblerLoss.hpp:32-43
 *   6  loss/HingeLoss.hpp:31-99                 7  the same with Squared = true
 *   8  loss/MultiLabelHingeLoss.hpp:31-71       9  the same with Squared = true
 *   10 loss/MultiLabelLogLoss.hpp:37-76
 * kind | 0x100 is the loss wrapped in NegatedLoss (loss/NegatedLoss.hpp:41-46): both results negated.
 * ------------------------------------------------------------------------------------------- */
constexpr int LOSS_NEGATED = 0x100;

/* core/NumericUtils.hpp:42-49 with the default epsilons (the scalar type's machine epsilon) */
template<typename T>
bool almost_equal(T a, T b) {
	const T e = std::numeric_limits<T>::epsilon();
	const T diff = std::abs(a - b);
	if (diff <= e)
		return true;
	return diff <= std::max(std::abs(a), std::abs(b)) * e;
}

/* core/NumericUtils.hpp:62-65 */
template<typename T>
bool decidedly_greater(T a, T b) {
	return a > b && !almost_equal(a, b);
}

/* the index of the one in a one-hot row (loss/HingeLoss.hpp:38-48: the last element that almost equals 1);
 * -1 when there is none, which the reference asserts against */
template<typename T>
i64 one_hot_index(const T* y, i64 cs, i64 V) {
	i64 ind = -1;
	for (i64 j = 0; j < V; ++j)
		if (almost_equal<T>(y[cs * j], (T) 1))
			ind = j;
	return ind;
}

template<typename T>
int loss_function(int kind, i64 N, i64 Ts, i64 V, T eps, const T* out, const T* obj, T* losses) {
	const bool negated = (kind & LOSS_NEGATED) != 0;
	kind &= ~LOSS_NEGATED;
	if (kind < 0 || kind > 10 || (kind == 3 && V != 1))
		return 1;
	std::vector<T> e((size_t) V);
	for (i64 n = 0; n < N; ++n)
		losses[n] = 0;
	for (i64 t = 0; t < Ts; ++t)
		for (i64 n = 0; n < N; ++n) {
			const T* o = out + n + N * t;
			const T* y = obj + n + N * t;
			const i64 cs = N * Ts;
			T l = 0;
			switch (kind) {
			case 0:
				for (i64 j = 0; j < V; ++j)
					l += (o[cs * j] - y[cs * j]) * (o[cs * j] - y[cs * j]);
				break;
			case 1: {
				T mx = o[0];
				for (i64 j = 1; j < V; ++j)
					mx = std::max(mx, o[cs * j]);
				T sum = 0;
				for (i64 j = 0; j < V; ++j) {
					e[j] = std::exp(o[cs * j] - mx);
					sum += e[j];
				}
				for (i64 j = 0; j < V; ++j)
					l += std::log(e[j] / (sum + eps)) * y[cs * j];
				l = -l;
				break;
			}
			case 2:
				for (i64 j = 0; j < V; ++j)
					l += std::abs(o[cs * j] - y[cs * j]);
				break;
			case 3:
				l = -(y[0] * std::log(o[0] + eps) + ((T) 1 - y[0]) * std::log((T) (1 + eps) - o[0]));
				break;
			case 4:
				for (i64 j = 0; j < V; ++j)
					l += std::log(o[cs * j] + eps) * y[cs * j];
				l = -l;
				break;
			case 5:
				for (i64 j = 0; j < V; ++j)
					l += std::log(o[cs * j] / (y[cs * j] + eps) + eps) * y[cs * j];
				l = -l;
				break;
			case 6:
			case 7: {
				const i64 c = one_hot_index<T>(y, cs, V);
				if (c < 0)
					return 2;
				const T score = o[cs * c];
				for (i64 j = 0; j < V; ++j) {
					if (j == c)
						continue;
					const T lj = std::max((T) 0, (T) (o[cs * j] - score + 1));
					l += kind == 7 ? lj * lj : lj;
				}
				break;
			}
			case 8:
			case 9:
				for (i64 j = 0; j < V; ++j) {
					const T lj = std::max((T) 0, (T) 1 - y[cs * j] * o[cs * j]);
					l += kind == 9 ? lj * lj : lj;
				}
				break;
			default:
				for (i64 j = 0; j < V; ++j)
					l += y[cs * j] * std::log(o[cs * j] + eps) + (1 - y[cs * j]) * std::log(1 + eps - o[cs * j]);
				break;
			}
			losses[n] += negated ? -l : l;
		}
	return 0;
}

/* grad = scale * d_function; scale = 1 / batch_size is SGDOptimizer::_train's division
 * (optimizer/SGDOptimizer.hpp:54-55). */
template<typename T>
int loss_d_function(int kind, i64 N, i64 Ts, i64 V, T eps, T scale, const T* out, const T* obj, T* grad) {
	if ((kind & LOSS_NEGATED) != 0) {
		scale = -scale;
		kind &= ~LOSS_NEGATED;
	}
	if (kind < 0 || kind > 10 || (kind == 3 && V != 1))
		return 1;
	std::vector<T> e((size_t) V);
	const i64 cs = N * Ts;
	for (i64 t = 0; t < Ts; ++t)
		for (i64 n = 0; n < N; ++n) {
			const i64 base = n + N * t;
			const T* o = out + base;
			const T* y = obj + base;
			T* g = grad + base;
			switch (kind) {
			case 0:
				for (i64 j = 0; j < V; ++j)
					g[cs * j] = scale * (2 * (o[cs * j] - y[cs * j]));
				break;
			case 1: {
				T mx = o[0];
				for (i64 j = 1; j < V; ++j)
					mx = std::max(mx, o[cs * j]);
				T sum = 0;
				for (i64 j = 0; j < V; ++j) {
					e[j] = std::exp(o[cs * j] - mx);
					sum += e[j];
				}
				for (i64 j = 0; j < V; ++j)
					g[cs * j] = scale * (e[j] / (sum + eps) - y[cs * j]);
				break;
			}
			case 2:
				for (i64 j = 0; j < V; ++j)
					g[cs * j] = scale * (T) (o[cs * j] - y[cs * j] >= 0 ? 1 : -1);
				break;
			case 3:
				g[0] = scale * -(y[0] / (o[0] + eps) - ((T) 1 - y[0]) / ((T) (1 + eps) - o[0]));
				break;
			case 4:
			case 5:
				for (i64 j = 0; j < V; ++j)
					g[cs * j] = scale * (-y[cs * j] / (o[cs * j] + eps));
				break;
			case 6:
			case 7: {
				const i64 c = one_hot_index<T>(y, cs, V);
				if (c < 0)
					return 2;
				const T score = o[cs * c];
				T total = 0;
				for (i64 j = 0; j < V; ++j) {
					if (j == c)
						continue;
					const T margin = o[cs * j] - score + 1;
					if (decidedly_greater<T>(margin, (T) 0)) {
						const T gj = kind == 7 ? 2 * margin : 1;
						total += gj;
						g[cs * j] = scale * gj;
					} else
						g[cs * j] = scale * (T) 0;
				}
				g[cs * c] = scale * -total;
				break;
			}
			case 8:
			case 9:
				for (i64 j = 0; j < V; ++j) {
					const T margin = 1 - y[cs * j] * o[cs * j];
					if (decidedly_greater<T>(margin, (T) 0))
						g[cs * j] = scale * (kind == 9 ? 2 * o[cs * j] - 2 * y[cs * j] : -y[cs * j]);
					else
						g[cs * j] = scale * (T) 0;
				}
				break;
			default:
				for (i64 j = 0; j < V; ++j) {
					T oj = o[cs * j];
					const T denominator = oj * (1 - oj);
					if (oj == 0)
						oj += eps;
					g[cs * j] = scale * ((y[cs * j] - oj) / denominator);
				}
				break;
			}
		}
	return 0;
}

/* ---------------------------------------------------------------------------------------------
 * DropoutLayer (layer/DropoutLayer.hpp:74-96). The reference draws its uniform numbers from Eigen's
 * generator (in.random(), :79), whose stream cannot be restated; the mask is a function of those
 * numbers, mask = (u <= dropout_prob ? 0 : 1 / (1 - dropout_prob + epsilon)), and both passes multiply
 * by it. Here the numbers come from splitmix64 (Steele, Lea, Flood 2014; Vigna's public-domain
 * splitmix64.c): pass number q of a layer seeded with s uses key = the q-th output of the stream seeded
 * with s, and the elements of the batch tensor (linear index i, sample index fastest) take the outputs of the
 * stream seeded with that key: a double the top 53 bits of output i, a float 24 bits of output i / 2 (bits 63..40
 * for even i, bits 31..8 for odd i), scaled to [0, 1).
 * ------------------------------------------------------------------------------------------- */
typedef unsigned long long u64;

u64 splitmix64_output(u64 seed, u64 index) {
	u64 z = seed + (index + 1) * 0x9E3779B97F4A7C15ull;
	z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
	z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
	return z ^ (z >> 31);
}

/* float: one output serves two elements, bits 63..40 the even one, bits 31..8 the odd one */
float dropout_uniform(u64 key, u64 i, float) {
	const u64 bits = splitmix64_output(key, i >> 1);
	return (float) ((i & 1) ? (bits >> 8) & 0xFFFFFFull : bits >> 40) * (1.0f / 16777216.0f);
}
double dropout_uniform(u64 key, u64 i, double) {
	return (double) (splitmix64_output(key, i) >> 11) * (1.0 / 9007199254740992.0);
}

template<typename T>
int dropout_uniforms(u64 seed, u64 pass, i64 n, T* u) {
	const u64 key = splitmix64_output(seed, pass);
	for (i64 i = 0; i < n; ++i)
		u[i] = dropout_uniform(key, (u64) i, T());
	return 0;
}

/* y = x * mask(u): the forward pass on the input, the backward pass on the output gradient (:82, :95) */
template<typename T>
int dropout_apply(i64 n, T prob, T eps, const T* u, const T* x, T* y) {
	const T scaling_factor = (T) 1 / (1 - prob + eps);
	for (i64 i = 0; i < n; ++i)
		y[i] = x[i] * (T) (u[i] <= prob ? 0 : scaling_factor);
	return 0;
}

/* ---------------------------------------------------------------------------------------------
 * BroadcastLayer (layer/BroadcastLayer.hpp:69-101): the input repeated bh x bw x bc times along its three
 * ranks (Eigen's broadcast: out(n, h, w, c) = in(n, h mod H, w mod W, c mod C)); backward sums the
 * replicas rank by rank, first rank first, each sum starting from zero and taking the slices in order.
 * ------------------------------------------------------------------------------------------- */
template<typename T>
int broadcast_forward(i64 N, i64 H, i64 W, i64 C, i64 bh, i64 bw, i64 bc, const T* x, T* out) {
	const i64 OH = H * bh, OW = W * bw, OC = C * bc;
	for (i64 c = 0; c < OC; ++c)
		for (i64 w = 0; w < OW; ++w)
			for (i64 h = 0; h < OH; ++h)
				for (i64 n = 0; n < N; ++n)
					out[n + N * (h + OH * (w + OW * c))] = x[n + N * ((h % H) + H * ((w % W) + W * (c % C)))];
	return 0;
}

template<typename T>
int broadcast_backward(i64 N, i64 H, i64 W, i64 C, i64 bh, i64 bw, i64 bc, const T* out_grad, T* in_grad) {
	i64 dims[4] = { N, H * bh, W * bw, C * bc };           /* of the tensor being reduced */
	const i64 in_dims[4] = { N, H, W, C }, reps[4] = { 1, bh, bw, bc };
	std::vector<T> cur(out_grad, out_grad + dims[0] * dims[1] * dims[2] * dims[3]);
	for (int r = 1; r < 4; ++r) {
		if (reps[r] <= 1)
			continue;
		i64 nd[4] = { dims[0], dims[1], dims[2], dims[3] };
		nd[r] = in_dims[r];
		std::vector<T> work((size_t) (nd[0] * nd[1] * nd[2] * nd[3]), (T) 0);
		for (i64 j = 0; j < reps[r]; ++j)
			for (i64 c = 0; c < nd[3]; ++c)
				for (i64 w = 0; w < nd[2]; ++w)
					for (i64 h = 0; h < nd[1]; ++h)
						for (i64 n = 0; n < nd[0]; ++n) {
							i64 src[4] = { n, h, w, c };
							src[r] += j * in_dims[r];
							work[n + nd[0] * (h + nd[1] * (w + nd[2] * c))] +=
									cur[src[0] + dims[0] * (src[1] + dims[1] * (src[2] + dims[2] * src[3]))];
						}
		cur.swap(work);
		dims[r] = nd[r];
	}
	std::copy(cur.begin(), cur.end(), in_grad);
	return 0;
}

/* ParameterRegularization::function and d_function for L1 (l2 = 0; parameter_regularization/L1ParameterRegularization.hpp:32-37),
 * L2 (l1 = 0; L2ParameterRegularization.hpp:32-37) and elastic net (ElasticNetParameterRegularization.hpp:36-42):
 * penalty = l1 sum |v| + 0.5 l2 sum v^2; gradient = (v >= 0 ? l1 : -l1) + v l2, which Parameters::regularize adds to the
 * gradient before the update (parameters/StandardParameters.hpp:133-136). */
template<typename T>
int regularization(i64 n, T l1, T l2, const T* values, T* penalty, T* grad) {
	T abs_sum = 0, sq_sum = 0;
	for (i64 i = 0; i < n; ++i) {
		abs_sum += std::abs(values[i]);
		sq_sum += values[i] * values[i];
		const T sign_term = values[i] >= 0 ? l1 : -l1;
		grad[i] = l2 == 0 ? sign_term : (l1 == 0 ? values[i] * l2 : sign_term + values[i] * l2);
	}
	*penalty = (l1 != 0 ? abs_sum * l1 : (T) 0) + (l2 != 0 ? sq_sum * ((T) .5 * l2) : (T) 0);
	return 0;
}

/* optimizer/VanillaSGDOptimizer.hpp:38-43 */
template<typename T>
int sgd_update(i64 n, T lr, const T* grad, T* values) {
	for (i64 i = 0; i < n; ++i)
		values[i] = values[i] - grad[i] * lr;
	return 0;
}

/* optimizer/AdamOptimizer.hpp:66-82 (bias corrections carry the epsilon; epsilon sits inside the root) */
template<typename T>
int adam_update(i64 n, T lr, T d1, T d2, T eps, i64 timestep, const T* grad, T* m, T* v, T* values) {
	const T l1_corr = (T) 1 / (1 - std::pow(1 - d1, (T) (timestep + 1)) + eps);
	const T l2_corr = (T) 1 / (1 - std::pow(1 - d2, (T) (timestep + 1)) + eps);
	for (i64 i = 0; i < n; ++i) {
		m[i] = m[i] * (1 - d1) + grad[i] * d1;
		v[i] = v[i] * (1 - d2) + grad[i] * grad[i] * d2;
		values[i] = values[i] - (m[i] * (lr * l1_corr)) / std::sqrt(v[i] * l2_corr + eps);
	}
	return 0;
}

/* The remaining optimizers' _update_params bodies (rule numbering as in the tests' front end):
 * 1 MomentumSGDOptimizer.hpp:54-72, 2 NesterovMomentumSGDOptimizer.hpp:43-55, 3 AdaGradOptimizer.hpp:50-70,
 * 4 RMSPropOptimizer.hpp:43-47, 5 AdaDeltaOptimizer.hpp:53-67, 7 AdaMaxOptimizer.hpp:44-60,
 * 8 NadamOptimizer.hpp:44-65, 9 AMSGradOptimizer.hpp:48-66 (0 and 6 are the two functions above).
 * h holds the optimizer's constructor arguments in their order; s0..s2 its state matrices. */
template<typename T>
int optimizer_update(int rule, const double* hd, i64 epoch, i64 timestep, i64 n, const T* grad, T* s0, T* s1, T* s2,
		T* values) {
	const T h0 = (T) hd[0], h1 = (T) hd[1], h2 = (T) hd[2], h3 = (T) hd[3];
	if (rule == 0)
		return sgd_update<T>(n, h0, grad, values);
	if (rule == 6)
		return adam_update<T>(n, h0, h1, h2, h3, timestep, grad, s0, s1, values);
	if (rule == 1 || rule == 2) {
		const T lr = h0 / (1 + h1 * epoch);
		for (i64 i = 0; i < n; ++i) {
			if (rule == 1) {
				s0[i] = s0[i] * h2 + grad[i] * lr;
				values[i] = values[i] - s0[i];
			} else {
				const T old = s0[i];
				s0[i] = old * h2 - grad[i] * lr;
				values[i] = values[i] + old * -h2 + s0[i] * (1 + h2);
			}
		}
		return 0;
	}
	if (rule == 3 || rule == 4) {
		const T eps = rule == 3 ? h1 : h2;
		for (i64 i = 0; i < n; ++i) {
			if (rule == 3)
				s0[i] += grad[i] * grad[i];
			else
				s0[i] = s0[i] * (1 - h1) + grad[i] * grad[i] * h1;
			values[i] = values[i] - grad[i] * h0 / (std::sqrt(s0[i]) + eps);
		}
		return 0;
	}
	if (rule == 5) {
		for (i64 i = 0; i < n; ++i) {
			s0[i] = s0[i] * (1 - h0) + grad[i] * grad[i] * h0;
			const T upd = -grad[i] * std::sqrt(s1[i] + h1) / std::sqrt(s0[i] + h1);
			values[i] = values[i] + upd;
			s1[i] = s1[i] * (1 - h0) + upd * upd * h0;
		}
		return 0;
	}
	if (rule == 7 || rule == 8 || rule == 9) {
		const T l1_corr = (T) 1 / (1 - std::pow(1 - h1, (T) (timestep + 1)) + h3);
		const T l1_next_corr = (T) 1 / (1 - std::pow(1 - h1, (T) (timestep + 2)) + h3);
		const T l2_corr = (T) 1 / (1 - std::pow(1 - h2, (T) (timestep + 1)) + h3);
		for (i64 i = 0; i < n; ++i) {
			s0[i] = s0[i] * (1 - h1) + grad[i] * h1;
			if (rule == 7) {
				s1[i] = std::max(s1[i] * (1 - h2), std::abs(grad[i]));
				values[i] = values[i] - (s0[i] * (h0 * l1_corr)) / (s1[i] + h3);
			} else {
				s1[i] = s1[i] * (1 - h2) + grad[i] * grad[i] * h2;
				if (rule == 8)
					values[i] = values[i] - ((grad[i] * (h1 * l1_corr) + s0[i] * ((1 - h1) * l1_next_corr)) * h0) /
							std::sqrt(s1[i] * l2_corr + h3);
				else {
					s2[i] = std::max(s1[i], s2[i]);
					values[i] = values[i] - (s0[i] * h0) / std::sqrt(s2[i] + h3);
				}
			}
		}
		return 0;
	}
	return 1;
}

} /* namespace */

#define CONV_ARGS i64 N, i64 H, i64 W, i64 C, i64 F, i64 RH, i64 RW, i64 pv, i64 ph, i64 sv, i64 sh, i64 dv, i64 dh
#define CONV_GEOM ConvGeom g = { N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh, 0, 0, 0, 0, 0, 0, 0, 0 }
#define POOL_ARGS i64 N, i64 H, i64 W, i64 C, i64 RH, i64 RW, i64 sv, i64 sh
#define POOL_GEOM PoolGeom g = { N, H, W, C, RH, RW, sv, sh, 0, 0 }

#define ORACLE_INSTANTIATE(T, SFX) \
extern "C" int oracle_conv_forward_##SFX(CONV_ARGS, const T* x, const T* w, const T* b, T* out, T* cache) { \
	CONV_GEOM; return conv_forward<T>(g, x, w, b, out, cache); } \
extern "C" int oracle_conv_backward_##SFX(CONV_ARGS, const T* cache, const T* w, const T* out_grad, T* wgrad, \
		T* bgrad, T* in_grad) { CONV_GEOM; return conv_backward<T>(g, cache, w, out_grad, wgrad, bgrad, in_grad); } \
extern "C" int oracle_dense_forward_##SFX(i64 N, i64 V, i64 O, const T* x, const T* w, const T* b, T* out) { \
	return dense_forward<T>(N, V, O, x, w, b, out); } \
extern "C" int oracle_dense_backward_##SFX(i64 N, i64 V, i64 O, const T* x, const T* w, const T* out_grad, \
		T* wgrad, T* bgrad, T* in_grad) { return dense_backward<T>(N, V, O, x, w, out_grad, wgrad, bgrad, in_grad); } \
extern "C" int oracle_bn_forward_##SFX(i64 groups, i64 L, const T* x, const T* gamma, const T* beta, T* avg_mean, \
		T* avg_inv_sd, int stats_init, int training, double decay, double eps, T* out, T* std_cache, T* inv_sd_cache) { \
	return bn_forward<T>(groups, L, x, gamma, beta, avg_mean, avg_inv_sd, stats_init, training, (T) decay, (T) eps, \
			out, std_cache, inv_sd_cache); } \
extern "C" int oracle_bn_backward_##SFX(i64 groups, i64 L, const T* out_grad, const T* gamma, const T* std_cache, \
		const T* inv_sd_cache, T* gamma_grad, T* beta_grad, T* in_grad) { \
	return bn_backward<T>(groups, L, out_grad, gamma, std_cache, inv_sd_cache, gamma_grad, beta_grad, in_grad); } \
extern "C" int oracle_act_forward_##SFX(int kind, i64 n, double p, const T* x, T* y) { \
	return act_forward<T>(kind, n, (T) p, x, y); } \
extern "C" int oracle_act_backward_##SFX(int kind, i64 n, double p, const T* x, const T* y, const T* g, T* dx) { \
	return act_backward<T>(kind, n, (T) p, x, y, g, dx); } \
extern "C" int oracle_softmax_forward_##SFX(i64 N, i64 V, double eps, const T* x, T* y) { \
	return softmax_forward<T>(N, V, (T) eps, x, y); } \
extern "C" int oracle_softmax_backward_##SFX(i64 N, i64 V, const T* y, const T* g, T* dx) { \
	return softmax_backward<T>(N, V, y, g, dx); } \
extern "C" int oracle_prelu_forward_##SFX(i64 N, i64 V, const T* alpha, const T* x, T* y) { \
	return prelu_forward<T>(N, V, alpha, x, y); } \
extern "C" int oracle_prelu_backward_##SFX(i64 N, i64 V, const T* alpha, const T* x, const T* g, T* ag, T* dx) { \
	return prelu_backward<T>(N, V, alpha, x, g, ag, dx); } \
extern "C" int oracle_pswish_forward_##SFX(i64 N, i64 V, const T* beta, const T* x, T* y) { \
	return pswish_forward<T>(N, V, beta, x, y); } \
extern "C" int oracle_pswish_backward_##SFX(i64 N, i64 V, const T* beta, const T* x, const T* g, T* bg, T* dx) { \
	return pswish_backward<T>(N, V, beta, x, g, bg, dx); } \
extern "C" int oracle_maxpool_forward_##SFX(POOL_ARGS, const T* x, T* out, unsigned* inds) { \
	POOL_GEOM; return maxpool_forward<T>(g, x, out, inds); } \
extern "C" int oracle_maxpool_backward_##SFX(POOL_ARGS, const T* out_grad, const unsigned* inds, T* in_grad) { \
	POOL_GEOM; return maxpool_backward<T>(g, out_grad, inds, in_grad); } \
extern "C" int oracle_meanpool_forward_##SFX(POOL_ARGS, const T* x, T* out) { \
	POOL_GEOM; return meanpool_forward<T>(g, x, out); } \
extern "C" int oracle_meanpool_backward_##SFX(POOL_ARGS, const T* out_grad, T* in_grad) { \
	POOL_GEOM; return meanpool_backward<T>(g, out_grad, in_grad); } \
extern "C" int oracle_transconv_forward_##SFX(CONV_ARGS, const T* x, const T* w, const T* b, T* out) { \
	TransGeom g = { N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh, 0, 0, 0, 0, 0, 0 }; \
	return transconv_forward<T>(g, x, w, b, out); } \
extern "C" int oracle_transconv_backward_##SFX(CONV_ARGS, const T* x, const T* w, const T* out_grad, T* wgrad, T* bgrad, \
		T* in_grad) { TransGeom g = { N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh, 0, 0, 0, 0, 0, 0 }; \
	return transconv_backward<T>(g, x, w, out_grad, wgrad, bgrad, in_grad); } \
extern "C" int oracle_dropout_uniforms_##SFX(unsigned long long seed, unsigned long long pass, i64 n, T* u) { \
	return dropout_uniforms<T>(seed, pass, n, u); } \
extern "C" int oracle_dropout_apply_##SFX(i64 n, double prob, double eps, const T* u, const T* x, T* y) { \
	return dropout_apply<T>(n, (T) prob, (T) eps, u, x, y); } \
extern "C" int oracle_broadcast_forward_##SFX(i64 N, i64 H, i64 W, i64 C, i64 bh, i64 bw, i64 bc, const T* x, T* out) { \
	return broadcast_forward<T>(N, H, W, C, bh, bw, bc, x, out); } \
extern "C" int oracle_broadcast_backward_##SFX(i64 N, i64 H, i64 W, i64 C, i64 bh, i64 bw, i64 bc, const T* g, T* dx) { \
	return broadcast_backward<T>(N, H, W, C, bh, bw, bc, g, dx); } \
extern "C" int oracle_loss_function_##SFX(int kind, i64 N, i64 Ts, i64 V, double eps, const T* out, const T* obj, T* losses) { \
	return loss_function<T>(kind, N, Ts, V, (T) eps, out, obj, losses); } \
extern "C" int oracle_loss_d_function_##SFX(int kind, i64 N, i64 Ts, i64 V, double eps, double scale, const T* out, \
		const T* obj, T* grad) { return loss_d_function<T>(kind, N, Ts, V, (T) eps, (T) scale, out, obj, grad); } \
extern "C" int oracle_regularization_##SFX(i64 n, double l1, double l2, const T* values, T* penalty, T* grad) { \
	return regularization<T>(n, (T) l1, (T) l2, values, penalty, grad); } \
extern "C" int oracle_sgd_update_##SFX(i64 n, double lr, const T* grad, T* values) { \
	return sgd_update<T>(n, (T) lr, grad, values); } \
extern "C" int oracle_optimizer_update_##SFX(int rule, const double* h, i64 epoch, i64 timestep, i64 n, const T* grad, T* s0, \
		T* s1, T* s2, T* values) { return optimizer_update<T>(rule, h, epoch, timestep, n, grad, s0, s1, s2, values); } \
extern "C" int oracle_adam_update_##SFX(i64 n, double lr, double d1, double d2, double eps, i64 timestep, const T* grad, \
		T* m, T* v, T* values) { return adam_update<T>(n, (T) lr, (T) d1, (T) d2, (T) eps, timestep, grad, m, v, values); }

ORACLE_INSTANTIATE(float, f32)
ORACLE_INSTANTIATE(double, f64)

extern "C" unsigned long long oracle_splitmix64_output(unsigned long long seed, unsigned long long index) {
	return splitmix64_output(seed, index);
}

extern "C" int oracle_num_threads(void) {
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

extern "C" void oracle_set_num_threads(int n) {
#ifdef _OPENMP
	/* core/EigenProxy.hpp:102-105 clamps the requested count to [1, hardware concurrency]. */
	const int hw = omp_get_num_procs();
	omp_set_num_threads(n < 1 ? 1 : (n > hw ? hw : n));
#else
	(void) n;
#endif
}
