/*
 * gemm_kernels.hip — MFMA implicit-GEMM kernels for the convolution and dense layers (gfx950).
 *
 * All tensors keep the reference's column-major (N,H,W,C) layout (N fastest), so a GEMM row index
 * m = n + N*(oh + OH*ow) walks contiguous memory and the patch matrix of
 * layer/kernel/ConvKernelLayer.hpp:125-142 never has to exist: its element A(m,k) is gathered
 * straight from the activation tensor into LDS.
 *
 *   gather_gemm_kernel   out[M x F] = A[M x K] * Wt[K x F] (+ bias)     forward and input gradient
 *   wgrad_kernel         P_s[K x F] = A_s^T * G_s over a slice s of M    weight gradient partials
 *   reduce_partials      dW += sum_s P_s in fixed order                 deterministic, no atomics
 *   colsum kernels       db += column sums of G                         bias gradient
 *
 * MFMA operand convention used throughout: the matrix instruction computes D[i][j] += A[i][k]*B[k][j]
 * with lane l holding A[i = l % TL][k = l / TL] and B[k = l / TL][j = l % TL]; accumulator register r
 * of lane l is D[i = acc_row(r, l / TL)][j = l % TL] (acc_row below). The j index is always mapped to the memory-
 * contiguous index of the output so that stores are coalesced.
 */
#include "common.hpp"

#include <algorithm>
#include <type_traits>

namespace cattle_hip {

namespace {

template<typename T> struct Mfma;

template<> struct Mfma<float> {
	static constexpr int TL = 32;   /* tile edge */
	static constexpr int KS = 2;    /* reduction slots per instruction */
	static constexpr int NACC = 16; /* accumulator registers per lane */
	typedef float acc_t __attribute__((ext_vector_type(16)));
	static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) {
		return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
	}
};

template<> struct Mfma<double> {
	static constexpr int TL = 16;
	static constexpr int KS = 4;
	static constexpr int NACC = 4;
	typedef double acc_t __attribute__((ext_vector_type(4)));
	static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) {
		return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
	}
};

/* Row (i index) of accumulator register r for a lane in reduction slot lk (= lane / TL), as measured
 * on gfx950: 32x32x2 f32 packs rows in groups of four per slot, 16x16x4 f64 interleaves the slots. */
template<typename T>
__device__ __forceinline__ int acc_row(int r, int lk) {
	if (std::is_same<T, float>::value)
		return (r / 4) * 8 + 4 * lk + (r % 4);
	return 4 * r + lk;
}

template<typename T, int V> struct VecOf { typedef T type __attribute__((ext_vector_type(V))); };
template<typename T> struct VecOf<T, 1> { typedef T type; };

template<typename T, int V>
__device__ __forceinline__ void vec_load(T (&dst)[V], const T* p) {
	if constexpr (V == 1) {
		dst[0] = *p;
	} else {
		typedef typename VecOf<T, V>::type vt;
		const vt v = *reinterpret_cast<const vt*>(p);
		#pragma unroll
		for (int i = 0; i < V; ++i)
			dst[i] = v[i];
	}
}

template<typename T, int V>
__device__ __forceinline__ void vec_store(T* p, const T (&src)[V]) {
	if constexpr (V == 1) {
		*p = src[0];
	} else {
		typedef typename VecOf<T, V>::type vt;
		vt v;
		#pragma unroll
		for (int i = 0; i < V; ++i)
			v[i] = src[i];
		*reinterpret_cast<vt*>(p) = v;
	}
}

/* Blocks are dealt round-robin to the 8 XCDs, each with its own L2; remap so that every XCD works
 * on one contiguous range of tiles and neighbouring tiles (which share input rows) share an L2. */
__device__ __forceinline__ int xcd_tile(int bid, int ntiles) {
	constexpr int XCDS = 8;
	const int per = (ntiles + XCDS - 1) / XCDS;
	return (bid % XCDS) * per + bid / XCDS;
}

/* ------------------------------------------------------------------------------------------------
 * out[M x F] = gather(src)[M x K] * wt[K x F] (+ bias).
 * Block tile BM x BF, wave tile WT_M x WT_F, reduction chunks of KC staged through double-buffered
 * LDS: As[k][m] (m fastest, exactly as it lies in memory) and Bs[k][f].
 * VEC = elements per global load along m (needs N % VEC == 0 and a 16-byte aligned src).
 * DIVS = the gather has divisors (strided input gradient).
 * ---------------------------------------------------------------------------------------------- */
template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int VEC, bool DIVS>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_F)
void gather_gemm_kernel(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias,
		T* __restrict__ out, const GatherGeom g, const int mtiles) {
	typedef Mfma<T> MF;
	constexpr int THREADS = 64 * WAVES_M * WAVES_F;
	constexpr int BM = WAVES_M * WT_M, BF = WAVES_F * WT_F;
	constexpr int PAD = std::is_same<T, float>::value ? 32 : 16;
	constexpr int LDA = BM + PAD, LDB = BF + PAD;
	constexpr int TL = MF::TL, KS = MF::KS;
	constexpr int MB = WT_M / TL, FB = WT_F / TL;
	constexpr int ACOLS = BM / VEC, ARP = THREADS / ACOLS, ASLOTS = KC / ARP;
	constexpr int VB = 16 / (int) sizeof(T);
	constexpr int BCOLS = BF / VB, BVECS = KC * BCOLS, BITER = (BVECS + THREADS - 1) / THREADS;
	static_assert(THREADS % ACOLS == 0 && KC % ARP == 0 && ASLOTS >= 1, "A loader mapping");
	static_assert(KC % KS == 0 && WT_M % TL == 0 && WT_F % TL == 0, "tile shape");

	__shared__ T As[2][KC][LDA];
	__shared__ T Bs[2][KC][LDB];

	const int tile = xcd_tile(blockIdx.x, mtiles);
	if (tile >= mtiles)
		return;
	const int tid = threadIdx.x;
	const int m0 = tile * BM;
	const int f0 = blockIdx.y * BF;

	/* --- per-thread gather state: a fixed group of VEC rows m, and a walking k row --- */
	const int acol = tid % ACOLS, arow0 = tid / ACOLS;
	const int m = m0 + acol * VEC;
	const bool mvalid = m < g.M;
	int n, ya0, yb0;
	{
		n = m % g.N;
		const int t = m / g.N;
		const int a = t % g.OA, b = t / g.OA;
		ya0 = a * g.SA + g.PA;
		yb0 = b * g.SB + g.PB;
	}
	int kr = arow0 % g.R, ks, kch;
	{
		const int t = arow0 / g.R;
		ks = t % g.S;
		kch = t / g.S;
	}
	const int eR = ARP % g.R, eS = (ARP / g.R) % g.S, eCh = (ARP / g.R) / g.S;

	T areg[ASLOTS][VEC];
	T breg[BITER][VB];

	auto load_tiles = [&](int k0) {
		#pragma unroll
		for (int s = 0; s < ASLOTS; ++s) {
			int ya = ya0 + kr * g.RA, yb = yb0 + ks * g.RB;
			bool ok = mvalid && kch < g.LC;
			if (DIVS) {
				const int qa = ya / g.DA, qb = yb / g.DB;
				ok = ok && qa * g.DA == ya && qb * g.DB == yb;
				ya = qa;
				yb = qb;
			}
			ok = ok && (unsigned) ya < (unsigned) g.LH && (unsigned) yb < (unsigned) g.LW;
			if (ok) {
				vec_load<T, VEC>(areg[s], src + (n + g.N * (ya + g.LH * (yb + g.LW * kch))));
			} else {
				#pragma unroll
				for (int v = 0; v < VEC; ++v)
					areg[s][v] = (T) 0;
			}
			/* advance the k row by ARP with carries */
			kr += eR;
			const int c1 = kr >= g.R;
			kr -= c1 ? g.R : 0;
			ks += eS + c1;
			const int c2 = ks >= g.S;
			ks -= c2 ? g.S : 0;
			kch += eCh + c2;
		}
		#pragma unroll
		for (int it = 0; it < BITER; ++it) {
			const int idx = tid + it * THREADS;
			if (BVECS % THREADS == 0 || idx < BVECS) {
				const int brow = idx / BCOLS, bcol = idx % BCOLS;
				vec_load<T, VB>(breg[it], wt + ((size_t) (k0 + brow) * g.ldw + f0 + bcol * VB));
			}
		}
	};
	auto store_tiles = [&](int buf) {
		#pragma unroll
		for (int s = 0; s < ASLOTS; ++s)
			vec_store<T, VEC>(&As[buf][arow0 + s * ARP][acol * VEC], areg[s]);
		#pragma unroll
		for (int it = 0; it < BITER; ++it) {
			const int idx = tid + it * THREADS;
			if (BVECS % THREADS == 0 || idx < BVECS) {
				const int brow = idx / BCOLS, bcol = idx % BCOLS;
				vec_store<T, VB>(&Bs[buf][brow][bcol * VB], breg[it]);
			}
		}
	};

	const int lane = tid % 64, wave = tid / 64;
	const int wm = wave % WAVES_M, wf = wave / WAVES_M;
	const int lc = lane % TL, lk = lane / TL;

	typename MF::acc_t acc[FB][MB];
	#pragma unroll
	for (int i = 0; i < FB; ++i)
		#pragma unroll
		for (int j = 0; j < MB; ++j)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r)
				acc[i][j][r] = (T) 0;

	const int nchunks = (g.K + KC - 1) / KC;
	load_tiles(0);
	store_tiles(0);
	__syncthreads();
	for (int c = 0; c < nchunks; ++c) {
		const int buf = c & 1;
		if (c + 1 < nchunks)
			load_tiles((c + 1) * KC);
		#pragma unroll
		for (int kk = 0; kk < KC; kk += KS) {
			T xa[MB], wb[FB];
			#pragma unroll
			for (int j = 0; j < MB; ++j)
				xa[j] = As[buf][kk + lk][wm * WT_M + j * TL + lc];
			#pragma unroll
			for (int i = 0; i < FB; ++i)
				wb[i] = Bs[buf][kk + lk][wf * WT_F + i * TL + lc];
			#pragma unroll
			for (int i = 0; i < FB; ++i)
				#pragma unroll
				for (int j = 0; j < MB; ++j)
					acc[i][j] = MF::mma(wb[i], xa[j], acc[i][j]);
		}
		if (c + 1 < nchunks)
			store_tiles(buf ^ 1);
		__syncthreads();
	}

	/* epilogue: D rows are filters, D columns are m (contiguous in memory) */
	#pragma unroll
	for (int i = 0; i < FB; ++i) {
		#pragma unroll
		for (int r = 0; r < MF::NACC; ++r) {
			const int f = f0 + wf * WT_F + i * TL + acc_row<T>(r, lk);
			if (f < g.F) {
				const T bv = bias ? bias[f] : (T) 0;
				#pragma unroll
				for (int j = 0; j < MB; ++j) {
					const int mm = m0 + wm * WT_M + j * TL + lc;
					if (mm < g.M)
						out[(size_t) mm + (size_t) g.M * f] = acc[i][j][r] + bv;
				}
			}
		}
	}
}

/* ------------------------------------------------------------------------------------------------
 * Weight-gradient partials: P[k + K*f] = sum over this block's slice of m of A(m,k) * G(m,f).
 * The reduction index m is the contiguous one, so both operand tiles are staged as [row][m] and a
 * lane fetches VR consecutive m with one 16-byte LDS read; since a sum may be taken in any order,
 * MFMA step e pairs reduction slot lk with m = mm + lk*VR + e for both operands.
 * grid = (ktiles * ftiles, splits).
 * ---------------------------------------------------------------------------------------------- */
template<typename T, int WAVES_K, int WAVES_F, int WT_K, int WT_F, int MC, int VEC>
__global__ __launch_bounds__(64 * WAVES_K * WAVES_F)
void wgrad_kernel(const T* __restrict__ src, const T* __restrict__ og, T* __restrict__ partials,
		const GatherGeom g, const int ktiles, const int chunks_per_split) {
	typedef Mfma<T> MF;
	constexpr int THREADS = 64 * WAVES_K * WAVES_F;
	constexpr int BK = WAVES_K * WT_K, BF = WAVES_F * WT_F;
	constexpr int VR = 16 / (int) sizeof(T);
	constexpr int LDM = MC + VR;
	constexpr int TL = MF::TL, KS = MF::KS;
	constexpr int KB = WT_K / TL, FB = WT_F / TL;
	constexpr int COLS = MC / VEC, RP = THREADS / COLS;
	constexpr int XSLOTS = BK / RP, GSLOTS = BF / RP;
	static_assert(THREADS % COLS == 0 && BK % RP == 0 && BF % RP == 0, "loader mapping");
	static_assert(MC % (VR * KS) == 0, "reduction chunk");

	__shared__ __attribute__((aligned(16))) T Xs[2][BK][LDM];
	__shared__ __attribute__((aligned(16))) T Gs[2][BF][LDM];
	__shared__ int4 ktab[BK];      /* per k row: ya term, yb term, channel offset, valid */

	const int tid = threadIdx.x;
	const int k0 = (blockIdx.x % ktiles) * BK;
	const int f0 = (blockIdx.x / ktiles) * BF;
	const int chunk_begin = blockIdx.y * chunks_per_split;
	const int total_chunks = (g.M + MC - 1) / MC;
	const int chunk_end = min(chunk_begin + chunks_per_split, total_chunks);

	for (int i = tid; i < BK; i += THREADS) {
		const int k = k0 + i;
		const int r = k % g.R, t = k / g.R;
		const int s = t % g.S, ch = t / g.S;
		ktab[i] = make_int4(r * g.RA, s * g.RB, g.N * g.LH * g.LW * ch, k < g.K ? 1 : 0);
	}

	const int col = tid % COLS, row0 = tid / COLS;
	/* m state of this thread's vector: starts at the first chunk of the slice, advances by MC */
	int m = chunk_begin * MC + col * VEC;
	int n = m % g.N, a, b;
	{
		const int t = m / g.N;
		a = t % g.OA;
		b = t / g.OA;
	}
	const int eN = MC % g.N, eA = (MC / g.N) % g.OA, eB = (MC / g.N) / g.OA;

	T xreg[XSLOTS][VEC], greg[GSLOTS][VEC];

	auto load_tiles = [&]() {
		const bool mvalid = m < g.M;
		const int ya0 = a * g.SA + g.PA, yb0 = b * g.SB + g.PB;
		#pragma unroll
		for (int s = 0; s < XSLOTS; ++s) {
			const int4 ke = ktab[row0 + s * RP];
			const int ya = ya0 + ke.x, yb = yb0 + ke.y;
			const bool ok = mvalid && ke.w && (unsigned) ya < (unsigned) g.LH && (unsigned) yb < (unsigned) g.LW;
			if (ok) {
				vec_load<T, VEC>(xreg[s], src + (n + g.N * (ya + g.LH * yb) + ke.z));
			} else {
				#pragma unroll
				for (int v = 0; v < VEC; ++v)
					xreg[s][v] = (T) 0;
			}
		}
		#pragma unroll
		for (int s = 0; s < GSLOTS; ++s) {
			const int f = f0 + row0 + s * RP;
			if (mvalid && f < g.F) {
				vec_load<T, VEC>(greg[s], og + ((size_t) m + (size_t) g.M * f));
			} else {
				#pragma unroll
				for (int v = 0; v < VEC; ++v)
					greg[s][v] = (T) 0;
			}
		}
		/* advance m by MC with carries into (a, b) */
		m += MC;
		n += eN;
		const int c1 = n >= g.N;
		n -= c1 ? g.N : 0;
		a += eA + c1;
		const int c2 = a >= g.OA;
		a -= c2 ? g.OA : 0;
		b += eB + c2;
	};
	auto store_tiles = [&](int buf) {
		#pragma unroll
		for (int s = 0; s < XSLOTS; ++s)
			vec_store<T, VEC>(&Xs[buf][row0 + s * RP][col * VEC], xreg[s]);
		#pragma unroll
		for (int s = 0; s < GSLOTS; ++s)
			vec_store<T, VEC>(&Gs[buf][row0 + s * RP][col * VEC], greg[s]);
	};

	const int lane = tid % 64, wave = tid / 64;
	const int wk = wave % WAVES_K, wf = wave / WAVES_K;
	const int lc = lane % TL, lk = lane / TL;

	typename MF::acc_t acc[FB][KB];
	#pragma unroll
	for (int i = 0; i < FB; ++i)
		#pragma unroll
		for (int j = 0; j < KB; ++j)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r)
				acc[i][j][r] = (T) 0;

	__syncthreads();                  /* ktab visible */
	if (chunk_begin < chunk_end) {
		load_tiles();
		store_tiles(0);
	}
	__syncthreads();
	for (int c = chunk_begin; c < chunk_end; ++c) {
		const int buf = (c - chunk_begin) & 1;
		if (c + 1 < chunk_end)
			load_tiles();
		#pragma unroll
		for (int mm = 0; mm < MC; mm += VR * KS) {
			T ga[FB][VR], xb[KB][VR];
			#pragma unroll
			for (int i = 0; i < FB; ++i)
				vec_load<T, VR>(ga[i], &Gs[buf][wf * WT_F + i * TL + lc][mm + lk * VR]);
			#pragma unroll
			for (int j = 0; j < KB; ++j)
				vec_load<T, VR>(xb[j], &Xs[buf][wk * WT_K + j * TL + lc][mm + lk * VR]);
			#pragma unroll
			for (int e = 0; e < VR; ++e)
				#pragma unroll
				for (int i = 0; i < FB; ++i)
					#pragma unroll
					for (int j = 0; j < KB; ++j)
						acc[i][j] = MF::mma(ga[i][e], xb[j][e], acc[i][j]);
		}
		if (c + 1 < chunk_end)
			store_tiles(buf ^ 1);
		__syncthreads();
	}

	T* dst = partials + (size_t) blockIdx.y * ((size_t) g.K * g.F);
	#pragma unroll
	for (int i = 0; i < FB; ++i) {
		#pragma unroll
		for (int r = 0; r < MF::NACC; ++r) {
			const int f = f0 + wf * WT_F + i * TL + acc_row<T>(r, lk);
			if (f < g.F) {
				#pragma unroll
				for (int j = 0; j < KB; ++j) {
					const int k = k0 + wk * WT_K + j * TL + lc;
					if (k < g.K)
						dst[(size_t) k + (size_t) g.K * f] = acc[i][j][r];
				}
			}
		}
	}
}

/* dst[i] += sum_s partials[s][i], s ascending: the order is fixed, so results are reproducible. */
template<typename T>
__global__ void reduce_partials_kernel(const T* __restrict__ partials, T* __restrict__ dst, size_t count, int splits) {
	const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= count)
		return;
	T s = (T) 0;
	for (int p = 0; p < splits; ++p)
		s += partials[(size_t) p * count + i];
	dst[i] += s;
}

/* Block-wide sum with wavefront shuffles then LDS; every thread of the block must call it. */
template<typename T>
__device__ __forceinline__ T block_sum(T v, T* lds) {
	#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		v += __shfl_down(v, off, 64);
	const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
	if (lane == 0)
		lds[wave] = v;
	__syncthreads();
	T total = (T) 0;
	if (threadIdx.x == 0) {
		const int nw = (blockDim.x + 63) / 64;
		for (int w = 0; w < nw; ++w)
			total += lds[w];
	}
	__syncthreads();
	return total;        /* valid in thread 0 */
}

/* Column sums of G[M x F]: grid (splits, F); block (s, f) sums rows [s*span, (s+1)*span). */
template<typename T>
__global__ __launch_bounds__(256)
void colsum_partial_kernel(const T* __restrict__ G, T* __restrict__ ws, size_t M, size_t span) {
	__shared__ T lds[4];
	const size_t begin = (size_t) blockIdx.x * span;
	const size_t end = begin + span < M ? begin + span : M;
	const T* col = G + M * blockIdx.y;
	T s = (T) 0;
	for (size_t i = begin + threadIdx.x; i < end; i += 256)
		s += col[i];
	const T total = block_sum(s, lds);
	if (threadIdx.x == 0)
		ws[(size_t) blockIdx.y * gridDim.x + blockIdx.x] = total;
}

template<typename T>
__global__ void colsum_final_kernel(const T* __restrict__ ws, T* __restrict__ dst, int F, int splits) {
	const int f = blockIdx.x * blockDim.x + threadIdx.x;
	if (f >= F)
		return;
	T s = (T) 0;
	for (int p = 0; p < splits; ++p)
		s += ws[(size_t) f * splits + p];
	dst[f] += s;
}

/* Forward weights: wt[k][f] = w[k + K*f], zero-padded to Kp rows x ldw columns. */
template<typename T>
__global__ void prep_fwd_weights_kernel(const T* __restrict__ w, T* __restrict__ wt, int K, int F, int Kp, int ldw) {
	const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= (size_t) Kp * ldw)
		return;
	const int f = (int) (i % ldw), k = (int) (i / ldw);
	wt[i] = (k < K && f < F) ? w[(size_t) k + (size_t) K * f] : (T) 0;
}

/* Input-gradient weights: wt[k' = rh + RH*(rw + RW*f)][c] = w[rh + RH*(rw + RW*c) + K*f]. */
template<typename T>
__global__ void prep_dgrad_weights_kernel(const T* __restrict__ w, T* __restrict__ wt, int RHW, int C, int F, int Kp,
		int ldw) {
	const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= (size_t) Kp * ldw)
		return;
	const int c = (int) (i % ldw), kp = (int) (i / ldw);
	const int tap = kp % RHW, f = kp / RHW;
	wt[i] = (f < F && c < C) ? w[(size_t) (tap + RHW * c) + (size_t) (RHW * C) * f] : (T) 0;
}

int round_up(int v, int to) {
	return (v + to - 1) / to * to;
}

constexpr int WT_ROW_PAD = 16;     /* >= every KC */
constexpr int WT_COL_PAD = 128;    /* >= every BF */

template<typename T> struct GemmCfg;
template<> struct GemmCfg<float> { static constexpr int KC = 16, VEC = 4; };
template<> struct GemmCfg<double> { static constexpr int KC = 8, VEC = 2; };

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F>
void launch_gather_variant(const T* src, const T* wt, const T* bias, T* out, const GatherGeom& g, bool vec, bool divs) {
	constexpr int KC = GemmCfg<T>::KC, VEC = GemmCfg<T>::VEC;
	constexpr int BM = WAVES_M * WT_M, BF = WAVES_F * WT_F;
	const int mtiles = (g.M + BM - 1) / BM;
	dim3 grid((unsigned) round_up(mtiles, 8), (unsigned) ((g.F + BF - 1) / BF));
	dim3 block(64 * WAVES_M * WAVES_F);
	if (vec && !divs)
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false><<<grid, block, 0, stream()>>>(src, wt, bias, out, g, mtiles);
	else if (vec && divs)
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, true><<<grid, block, 0, stream()>>>(src, wt, bias, out, g, mtiles);
	else if (!divs)
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, 1, false><<<grid, block, 0, stream()>>>(src, wt, bias, out, g, mtiles);
	else
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, 1, true><<<grid, block, 0, stream()>>>(src, wt, bias, out, g, mtiles);
	CATTLE_HIP_CHECK(hipGetLastError());
}

template<typename T>
void launch_gather(const T* src, const T* wt, const T* bias, T* out, const GatherGeom& g) {
	const bool vec = g.N % GemmCfg<T>::VEC == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0;
	const bool divs = g.DA != 1 || g.DB != 1;
	if (std::is_same<T, float>::value) {
		if (g.F > 64)
			launch_gather_variant<T, 4, 2, 64, 64>(src, wt, bias, out, g, vec, divs);
		else if (g.F > 32)
			launch_gather_variant<T, 4, 1, 64, 64>(src, wt, bias, out, g, vec, divs);
		else
			launch_gather_variant<T, 4, 1, 64, 32>(src, wt, bias, out, g, vec, divs);
	} else {
		if (g.F > 32)
			launch_gather_variant<T, 4, 2, 64, 32>(src, wt, bias, out, g, vec, divs);
		else
			launch_gather_variant<T, 4, 1, 64, 32>(src, wt, bias, out, g, vec, divs);
	}
}

GatherGeom forward_geom(const ConvShape& s, int N) {
	GatherGeom g;
	g.N = N; g.LH = s.H; g.LW = s.W; g.LC = s.C;
	g.OA = s.OH(); g.OB = s.OW();
	g.R = s.RH; g.S = s.RW;
	g.SA = s.sv; g.SB = s.sh; g.RA = s.dv + 1; g.RB = s.dh + 1; g.PA = -s.pv; g.PB = -s.ph; g.DA = 1; g.DB = 1;
	g.M = N * g.OA * g.OB; g.K = s.K(); g.F = s.F;
	g.ldw = round_up(s.F, WT_COL_PAD);
	return g;
}

GatherGeom dgrad_geom(const ConvShape& s, int N) {
	GatherGeom g;
	g.N = N; g.LH = s.OH(); g.LW = s.OW(); g.LC = s.F;
	g.OA = s.H; g.OB = s.W;
	g.R = s.RH; g.S = s.RW;
	g.SA = 1; g.SB = 1; g.RA = -(s.dv + 1); g.RB = -(s.dh + 1); g.PA = s.pv; g.PB = s.ph; g.DA = s.sv; g.DB = s.sh;
	g.M = N * s.H * s.W; g.K = s.RH * s.RW * s.F; g.F = s.C;
	g.ldw = round_up(s.C, WT_COL_PAD);
	return g;
}

void check_sizes(const ConvShape& s, int N) {
	CATTLE_HIP_REQUIRE(N > 0, "batch size must be positive");
	const double lim = 2147483647.0;
	const double in_elems = (double) N * s.H * s.W * s.C, out_elems = (double) N * s.OH() * s.OW() * s.F;
	CATTLE_HIP_REQUIRE(in_elems <= lim && out_elems <= lim, "tensor exceeds 2^31-1 elements");
}

/* Split plan of the weight-gradient reduction over M. */
template<typename T> struct WgradCfg;
template<> struct WgradCfg<float> { static constexpr int WK = 2, WF = 2, TK = 64, TF = 64, MC = 32, VEC = 4; };
template<> struct WgradCfg<double> { static constexpr int WK = 2, WF = 2, TK = 32, TF = 32, MC = 32, VEC = 2; };

struct WgradPlan {
	int ktiles, ftiles, splits, chunks_per_split;
};

template<typename T>
WgradPlan wgrad_plan(int M, int K, int F) {
	typedef WgradCfg<T> C;
	WgradPlan p;
	p.ktiles = (K + C::WK * C::TK - 1) / (C::WK * C::TK);
	p.ftiles = (F + C::WF * C::TF - 1) / (C::WF * C::TF);
	const int chunks = (M + C::MC - 1) / C::MC;
	const int tiles = p.ktiles * p.ftiles;
	int want = std::max(1, (1024 + tiles - 1) / tiles);      /* about four blocks per CU */
	want = std::min(want, std::max(1, chunks / 8));           /* at least 8 chunks per block */
	p.chunks_per_split = (chunks + want - 1) / want;
	p.splits = (chunks + p.chunks_per_split - 1) / p.chunks_per_split;
	return p;
}

constexpr int COLSUM_MAX_SPLITS = 64;

int colsum_splits(size_t M, int F) {
	const size_t by_rows = std::max<size_t>(1, M / 4096);
	const size_t by_fill = std::max<size_t>(1, (size_t) 1024 / (size_t) std::max(1, F));
	return (int) std::min<size_t>(COLSUM_MAX_SPLITS, std::min(by_rows, by_fill));
}

} /* namespace */

template<typename T>
ConvWorkspace conv_workspace(const ConvShape& s, int N) {
	check_sizes(s, N);
	ConvWorkspace ws;
	ws.wt_fwd = (size_t) round_up(s.K(), WT_ROW_PAD) * round_up(s.F, WT_COL_PAD);
	ws.wt_dgrad = (size_t) round_up(s.RH * s.RW * s.F, WT_ROW_PAD) * round_up(s.C, WT_COL_PAD);
	const int M = N * s.OH() * s.OW();
	const WgradPlan p = wgrad_plan<T>(M, s.K(), s.F);
	ws.partials = (size_t) p.splits * s.K() * s.F + (size_t) COLSUM_MAX_SPLITS * s.F;
	return ws;
}

template<typename T>
void conv_forward(const ConvShape& s, int N, const T* x, const T* w, const T* b, T* out, T* wt, bool wt_ready) {
	check_sizes(s, N);
	const GatherGeom g = forward_geom(s, N);
	if (!wt_ready) {
		const int Kp = round_up(g.K, WT_ROW_PAD);
		const size_t count = (size_t) Kp * g.ldw;
		prep_fwd_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wt, g.K, g.F, Kp, g.ldw);
		CATTLE_HIP_CHECK(hipGetLastError());
	}
	launch_gather<T>(x, wt, b, out, g);
}

template<typename T>
void conv_backward(const ConvShape& s, int N, const T* x, const T* w, const T* out_grad, T* wgrad, T* bgrad,
		T* in_grad, T* wt_dgrad, bool wt_ready, T* partials) {
	check_sizes(s, N);
	typedef WgradCfg<T> C;
	const GatherGeom g = forward_geom(s, N);
	/* weight gradient: split-M partials, then a fixed-order reduction that accumulates into wgrad */
	{
		const WgradPlan p = wgrad_plan<T>(g.M, g.K, g.F);
		dim3 grid((unsigned) (p.ktiles * p.ftiles), (unsigned) p.splits);
		dim3 block(64 * C::WK * C::WF);
		const bool vec = N % C::VEC == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
				(reinterpret_cast<uintptr_t>(out_grad) & 15) == 0;
		if (vec)
			wgrad_kernel<T, C::WK, C::WF, C::TK, C::TF, C::MC, C::VEC><<<grid, block, 0, stream()>>>(x, out_grad, partials, g,
					p.ktiles, p.chunks_per_split);
		else
			wgrad_kernel<T, C::WK, C::WF, C::TK, C::TF, C::MC, 1><<<grid, block, 0, stream()>>>(x, out_grad, partials, g,
					p.ktiles, p.chunks_per_split);
		CATTLE_HIP_CHECK(hipGetLastError());
		const size_t count = (size_t) g.K * g.F;
		reduce_partials_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(partials, wgrad, count, p.splits);
		CATTLE_HIP_CHECK(hipGetLastError());
		/* bias gradient */
		T* bws = partials + (size_t) p.splits * count;
		const int cs = colsum_splits((size_t) g.M, g.F);
		const size_t span = ((size_t) g.M + cs - 1) / cs;
		colsum_partial_kernel<T><<<dim3((unsigned) cs, (unsigned) g.F), 256, 0, stream()>>>(out_grad, bws, (size_t) g.M, span);
		CATTLE_HIP_CHECK(hipGetLastError());
		colsum_final_kernel<T><<<(unsigned) ((g.F + 255) / 256), 256, 0, stream()>>>(bws, bgrad, g.F, cs);
		CATTLE_HIP_CHECK(hipGetLastError());
	}
	if (!in_grad)
		return;
	const GatherGeom d = dgrad_geom(s, N);
	if (!wt_ready) {
		const int Kp = round_up(d.K, WT_ROW_PAD);
		const size_t count = (size_t) Kp * d.ldw;
		prep_dgrad_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wt_dgrad, s.RH * s.RW, s.C, s.F,
				Kp, d.ldw);
		CATTLE_HIP_CHECK(hipGetLastError());
	}
	launch_gather<T>(out_grad, wt_dgrad, (const T*) nullptr, in_grad, d);
}

template ConvWorkspace conv_workspace<float>(const ConvShape&, int);
template ConvWorkspace conv_workspace<double>(const ConvShape&, int);
template void conv_forward<float>(const ConvShape&, int, const float*, const float*, const float*, float*, float*, bool);
template void conv_forward<double>(const ConvShape&, int, const double*, const double*, const double*, double*, double*, bool);
template void conv_backward<float>(const ConvShape&, int, const float*, const float*, const float*, float*, float*, float*,
		float*, bool, float*);
template void conv_backward<double>(const ConvShape&, int, const double*, const double*, const double*, double*, double*,
		double*, double*, bool, double*);

} /* namespace cattle_hip */
