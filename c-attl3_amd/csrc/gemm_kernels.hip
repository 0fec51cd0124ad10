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
 *                        (+ bias-gradient partials: column sums of G from the tile already in LDS)
 *   reduce_partials      dW += sum_s P_s, db += sum_s p_s in fixed order    deterministic, no atomics
 *
 * MFMA operand convention used throughout: the matrix instruction computes D[i][j] += A[i][k]*B[k][j]
 * with lane l holding A[i = l % TL][k = l / TL] and B[k = l / TL][j = l % TL]; accumulator register r
 * of lane l is D[i = acc_row(r, l / TL)][j = l % TL] (acc_row below). The j index is always mapped to the memory-
 * contiguous index of the output so that stores are coalesced.
 */
#include "common.hpp"
#include "act_math.hpp"
#include "lstm_math.hpp"

#include <algorithm>
#include <functional>
#include <limits>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <unistd.h>
#include <vector>

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

/* Reduction chunk, global-load vector width and LDS row padding of the gather GEMM. The padding
 * keeps the two (f32) or four (f64) reduction slots of a wave on different banks; the 512-row
 * tile uses the smaller padding that still does, so that two blocks fit the 160 KB of LDS. */
template<typename T> struct GemmCfg;
template<> struct GemmCfg<float> {
	static constexpr int KC = 16, VEC = 4;
	static constexpr int pad(int bm) { return bm >= 512 ? 16 : 32; }
};
template<> struct GemmCfg<double> {
	static constexpr int KC = 8, VEC = 2;
	static constexpr int pad(int) { return 16; }
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

/* The same from a pointer that is known to point to global memory. A pointer the compiler cannot place (the select
 * between the source tensor and the block of zeros, for one) makes it emit flat loads, and those count against the LDS
 * counter as well as the memory counter: every wait for an LDS read in the MFMA loop then also waits for the global
 * loads of the next chunk, which undoes the prefetch. */
template<typename T, int V>
__device__ __forceinline__ void vec_load_global(T (&dst)[V], const T* p) {
	if constexpr (V == 1) {
		dst[0] = *(const __attribute__((address_space(1))) T*) p;
	} else {
		typedef typename VecOf<T, V>::type vt;
		const vt v = *(const __attribute__((address_space(1))) vt*) p;
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

/* The same as a streaming store to global memory: results that the storing XCD will not read again need no place in
 * its L2, and a kernel's end does not wait for them to be written back from there. */
template<typename T, int V>
__device__ __forceinline__ void vec_store_stream(T* p, const T (&src)[V]) {
	if constexpr (V == 1) {
		__builtin_nontemporal_store(src[0], (__attribute__((address_space(1))) T*) p);
	} else {
		typedef typename VecOf<T, V>::type vt;
		vt v;
		#pragma unroll
		for (int i = 0; i < V; ++i)
			v[i] = src[i];
		__builtin_nontemporal_store(v, (__attribute__((address_space(1))) vt*) p);
	}
}

/* fn(std::integral_constant<int, 0>()) ... fn(std::integral_constant<int, N - 1>()): a loop whose index is a
 * compile-time constant in the body (register arrays indexed by it stay registers) */
template<int N, typename Fn>
__device__ __forceinline__ void static_for(Fn fn) {
	if constexpr (N > 0) {
		static_for<N - 1>(fn);
		fn(std::integral_constant<int, N - 1>());
	}
}

/* Blocks are dealt round-robin to the 8 XCDs, each with its own L2; remap so that every XCD works
 * on one contiguous range of tiles and neighbouring tiles (which share input rows) share an L2. */
__device__ __forceinline__ int xcd_tile(int bid, int ntiles) {
	constexpr int XCDS = 8;
	const int per = (ntiles + XCDS - 1) / XCDS;
	return (bid % XCDS) * per + bid / XCDS;
}

/* The M tiles of a convolution form a grid of `rows` tiles per output column times `cols` columns
 * (tile = r + rows*col) when a column is a whole number of tiles. Walking that grid column by
 * column makes the ~64 tiles an XCD runs at a time one or two tall columns, and the halo they
 * share with the next column is long gone from L2 when that column's turn comes (each input
 * element was fetched about three times). Walking it in bands of SWIZZLE_COLS columns, row by row,
 * makes the running set a compact block instead. Returns the tile for position q of the walk. */
constexpr int SWIZZLE_COLS = 8;
__device__ __forceinline__ int swizzle_tile(int q, int rows, int cols) {
	const int band = q / (rows * SWIZZLE_COLS);
	const int rem = q - band * rows * SWIZZLE_COLS;
	const int width = min(SWIZZLE_COLS, cols - band * SWIZZLE_COLS);
	const int r = rem / width;
	return r + rows * (band * SWIZZLE_COLS + rem - r * width);
}

/* Where gathered loads that fall into the zero padding are pointed at. */
__device__ __attribute__((aligned(16))) const unsigned g_zero_block[4] = { 0u, 0u, 0u, 0u };

/* ------------------------------------------------------------------------------------------------
 * out[M x F] = gather(src)[M x K] * wt[K x F] (+ bias).
 * Block tile BM x BF, wave tile WT_M x WT_F, reduction chunks of KC staged through double-buffered
 * LDS: As[k][m] (m fastest, exactly as it lies in memory) and Bs[k][f].
 *
 * Keeping the MFMA pipe fed means keeping other vector instructions out of the loop, so:
 *  - the per-k part of the gather (element offset, row/column displacement) comes from a small
 *    table in LDS that one wave keeps three chunks ahead; a thread only adds its own base;
 *  - loads that fall into the zero padding are redirected to a 16-byte block of zeros in device
 *    memory (a pointer select), so the load itself is unconditional: no branch, no zero fill;
 *  - a lane's MB column blocks are interleaved (column = MB*lane + j) so that its operand values
 *    are adjacent in LDS and in the output: one LDS read per operand and reduction step with an
 *    immediate offset, and one vector store per output row.
 * VEC = elements per global load along m (needs N % VEC == 0 and a 16-byte aligned src).
 * DIVS = the gather has divisors (strided input gradient).
 * ---------------------------------------------------------------------------------------------- */
/* How a launch covers the M tiles, which are walked in the order swizzle_tile defines. The first
 * main_count positions of the walk are whole tiles, one block each (blocks [0, main_blocks), dealt to the
 * XCDs in contiguous ranges). The remaining split_count positions have their reduction cut into ksplit
 * parts of chunks_per_part chunks, one block per part (blocks from main_blocks on, so they are dispatched
 * last and fill the chip as the whole tiles drain): such a block writes its BM x BF partial sums, without
 * bias, to `partials`, laid out [position - main_count][f block][part][f][m], and split_reduce_kernel adds
 * the parts in a fixed order. */
struct GatherLaunch {
	int mtiles, tile_rows;
	int main_count, main_blocks;
	int split_count, ksplit, chunks_per_part;
	int sample_blocks;      /* > 0: tile rows are blocks of SB samples x BM / SB positions, see tile_row_m */
	int pos_b;              /* blocked order: positions of a tile along b (the other BM / SB / pos_b lie along a) */
	int sb_shift;           /* log2 of SB, the samples per block of the blocked order: 5 except under a pooling epilogue */
};

/* Row `row` of M tile `tile` as an index m = n + N * (a + OA * b) of the GEMM. Plain order: the tile is BM
 * consecutive m (BM consecutive samples of one output position when N >= BM). Blocked order (sample_blocks =
 * N / SB > 0, needs N % SB == 0; SB = 32 unless a pooling epilogue picked fewer): the tile is SB samples of a pa x pos_b
 * rectangle of output positions (pa = BM / SB / pos_b along a, OA % pa == 0, OB % pos_b == 0), so that the receptor
 * fields of its rows overlap and a tile touches about half as many distinct input bytes; tiles of one strip of pos_b
 * columns are numbered sample block fastest, and tile_rows counts the tiles of a strip. Rows stay groups of SB
 * consecutive samples, so vector accesses along n are unaffected. */
__device__ __forceinline__ int tile_row_m(const GatherLaunch& L, const GatherGeom& g, int tile, int BM, int row, int sb_shift = 5) {
	if (L.sample_blocks == 0)
		return tile * BM + row;
	const int strip = tile / L.tile_rows, r = tile - strip * L.tile_rows;
	const int ab = r / L.sample_blocks, nb = r - ab * L.sample_blocks;
	const int pa = (BM >> sb_shift) / L.pos_b, p = row >> sb_shift;
	const int pb_i = p / pa, pa_i = p - pb_i * pa;
	return (nb << sb_shift) + (row & ((1 << sb_shift) - 1)) + g.N * (ab * pa + pa_i + g.OA * (strip * L.pos_b + pb_i));
}

/* Element offset of row m of the result in `out` (GatherGeom's output map); consecutive samples of one position stay
 * consecutive, so vector stores along n are unaffected. */
__device__ __forceinline__ size_t out_row(const GatherGeom& g, int m) {
	if (g.out_sa == 1 && g.out_sb == 1 && g.out_a0 == 0 && g.out_b0 == 0 && g.out_OA == g.OA)
		return (size_t) m;
	const int n = m % g.N, t = m / g.N;
	const int a = t % g.OA, b = t / g.OA;
	return (size_t) n + (size_t) g.N * (size_t) ((g.out_a0 + g.out_sa * a) + g.out_OA * (g.out_b0 + g.out_sb * b));
}

/* Sum of v over a group of TL consecutive lanes (TL = 16: a row of the wavefront; TL = 32: two rows) with data-parallel
 * primitives of the vector ALU - lane exchanges inside quads, mirrored halves of a row, the last lane of a row broadcast to
 * the next row - so that no step goes through the LDS crossbar, which the wavefronts of a CU share (a butterfly of
 * ds_bpermute over the 64 column sums of a lane was most of the moments epilogue's time). The total is valid in the
 * last lane of the group (for TL = 16 in all of them). */
template<int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v) {
	return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}
template<int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_move(double v) {
	const long long bits = __builtin_bit_cast(long long, v);
	const int lo = __builtin_amdgcn_update_dpp(0, (int) (bits & 0xffffffffll), CTRL, ROW_MASK, 0xF, false);
	const int hi = __builtin_amdgcn_update_dpp(0, (int) (bits >> 32), CTRL, ROW_MASK, 0xF, false);
	return __builtin_bit_cast(double, ((long long) hi << 32) | (long long) (unsigned) lo);
}
template<typename T, int TL>
__device__ __forceinline__ T lane_group_sum(T v) {
	static_assert(TL == 16 || TL == 32, "a row or two rows of the wavefront");
	v += dpp_move<0xB1, 0xF>(v);            /* quad_perm [1, 0, 3, 2] */
	v += dpp_move<0x4E, 0xF>(v);            /* quad_perm [2, 3, 0, 1] */
	v += dpp_move<0x141, 0xF>(v);           /* row_half_mirror */
	v += dpp_move<0x140, 0xF>(v);           /* row_mirror */
	if constexpr (TL == 32)
		v += dpp_move<0x142, 0xA>(v);       /* row_bcast:15 into rows 1 and 3 (the other rows receive zero) */
	return v;
}

/* Several gathered GEMMs of one source and one result tensor in a single launch (the residue classes of a strided
 * input gradient): blockIdx.z picks the problem, whose geometry, tile walk and prepared weights come from this table
 * instead of the kernel's own arguments. No cut reductions: every tile is whole. */
constexpr int MAX_GATHER_CLASSES = 9;
template<typename T> struct GatherClasses {
	GatherGeom g[MAX_GATHER_CLASSES];
	GatherLaunch L[MAX_GATHER_CLASSES];
	const T* wt[MAX_GATHER_CLASSES];
};

/* A block's place in the launch as the GEMM bodies see it: the kernels that run a body alone pass the hardware's block
 * index, a kernel that runs two problems in one launch passes each its own numbering. */
struct BlockPlace {
	int x, y, ny;           /* block index along x and y, blocks along y */
};
__device__ __forceinline__ BlockPlace own_block_place() {
	return BlockPlace{ (int) blockIdx.x, (int) blockIdx.y, (int) gridDim.y };
}

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int VEC, bool DIVS, int EPI, int PF>
__device__ __forceinline__ void gather_gemm_body(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias,
		T* __restrict__ out, const GatherGeom& g, const GatherLaunch& L, T* __restrict__ partials, const Epilogue<T>& E,
		const BlockPlace bp);

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int VEC, bool DIVS, int EPI = EPI_NONE, int PF = 1>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_F)
void gather_gemm_kernel(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias,
		T* __restrict__ out, const GatherGeom g, const GatherLaunch L, T* __restrict__ partials, const Epilogue<T> E) {
	gather_gemm_body<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, DIVS, EPI, PF>(src, wt, bias, out, g, L, partials, E, own_block_place());
}

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int VEC>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_F)
void gather_gemm_classes_kernel(const T* __restrict__ src, T* __restrict__ out, const GatherClasses<T> classes) {
	const GatherGeom g = classes.g[blockIdx.z];
	const GatherLaunch L = classes.L[blockIdx.z];
	const Epilogue<T> none = { 0, (T) 0, nullptr, nullptr, 1, 1, 1, 1, nullptr, {} };
	gather_gemm_body<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_NONE, 1>(src, classes.wt[blockIdx.z], (const T*) nullptr, out, g, L,
			(T*) nullptr, none, own_block_place());
}

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int VEC, bool DIVS, int EPI, int PF>
__device__ __forceinline__ void gather_gemm_body(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias,
		T* __restrict__ out, const GatherGeom& g, const GatherLaunch& L, T* __restrict__ partials, const Epilogue<T>& E,
		const BlockPlace bp) {
	typedef Mfma<T> MF;
	constexpr int THREADS = 64 * WAVES_M * WAVES_F;
	constexpr int BM = WAVES_M * WT_M, BF = WAVES_F * WT_F;
	constexpr int PAD = GemmCfg<T>::pad(BM);
	constexpr int LDA = BM + PAD, LDB = BF + PAD;
	constexpr int TL = MF::TL, KS = MF::KS;
	constexpr int MB = WT_M / TL, FB = WT_F / TL;
	constexpr int ACOLS = BM / VEC, ARP = THREADS / ACOLS, ASLOTS = KC / ARP;
	constexpr int VB = 16 / (int) sizeof(T);
	constexpr int BCOLS = BF / VB, BVECS = KC * BCOLS, BITER = (BVECS + THREADS - 1) / THREADS;
	constexpr int INVALID = -(1 << 30);
	static_assert(THREADS % ACOLS == 0 && KC % ARP == 0 && ASLOTS >= 1, "A loader mapping");
	static_assert(KC % KS == 0 && WT_M % TL == 0 && WT_F % TL == 0, "tile shape");
	static_assert(THREADS >= KC, "table writers");

	__shared__ __attribute__((aligned(32))) T As[2][KC][LDA];
	__shared__ __attribute__((aligned(32))) T Bs[2][KC][LDB];
	/* PF = how many chunks ahead of the MFMAs the global loads run (held in registers until their turn to be stored to
	 * LDS): 1 for the large tiles, whose chunk of MFMA work covers the latency of a load; more for the short tiles of
	 * small problems, where a chunk is a few hundred cycles of MFMAs and a load takes a thousand. */
	constexpr int NSLOT = PF + 2;
	__shared__ int4 ktab[NSLOT][KC];     /* per reduction index: element offset, ya term, yb term, channel offset */

	int local, part = 0;
	const bool split = bp.x >= L.main_blocks;
	if (!split) {
		local = xcd_tile(bp.x, L.main_count);
		if (local >= L.main_count)
			return;
	} else {
		const int r = bp.x - L.main_blocks;
		local = r / L.ksplit;
		part = r - local * L.ksplit;
		if (local >= L.split_count)
			return;
	}
	int tile = split ? L.main_count + local : local;
	if (L.tile_rows > 0)
		tile = swizzle_tile(tile, L.tile_rows, L.mtiles / L.tile_rows);
	const int tid = threadIdx.x;
	const int f0 = bp.y * BF;
	/* The bias values of the tile's columns go through LDS: fetched now, read in the epilogue, many barriers later.
	 * Read from global memory there, each of a lane's FB * NACC values was a load with a wait of its own in front
	 * of its store: sixteen to thirty-two memory round trips in a row at the end of every block. */
	static_assert(THREADS >= BF, "one thread per bias value");
	__shared__ T bias_s[BF];
	if (tid < BF) {
		const int fsrc = EPI == EPI_LSTM && f0 + tid < g.F ? lstm_gate_column(f0 + tid, BF / 4, g.F / 4) : f0 + tid;
		bias_s[tid] = (bias != nullptr && f0 + tid < g.F) ? bias[fsrc] : (T) 0;
	}
	/* this block's chunks of the reduction: all of them, or one part */
	const int chunk0 = split ? part * L.chunks_per_part : 0;
	const int nchunks = split ? min(L.chunks_per_part, (g.K + KC - 1) / KC - chunk0) : (g.K + KC - 1) / KC;

	/* EPI_LSTM: this thread's state elements - LV consecutive rows (samples) of one hidden channel of the tile's CB per
	 * group, so that every tensor of the step is read and written LV elements at a time - and what their forward step
	 * reads besides this kernel's own sums, fetched now and used in the epilogue */
	constexpr int CB = BF / 4, LSTM_ELEMS = EPI == EPI_LSTM ? BM * CB / THREADS : 1;
	constexpr int LV = EPI == EPI_LSTM && BM * CB % (THREADS * VEC) == 0 ? VEC : 1, LSTM_GROUPS = LSTM_ELEMS / LV;
	unsigned lstm_e[LSTM_GROUPS];
	LstmForwardInputs<T> lstm_in[LSTM_GROUPS][LV];
	if constexpr (EPI == EPI_LSTM) {
		static_assert(BM * CB % THREADS == 0, "whole rounds of threads over a tile's state elements");
		#pragma unroll
		for (int gi = 0; gi < LSTM_GROUPS; ++gi) {
			const int idx = tid + gi * THREADS, row = (idx % (BM / LV)) * LV, cl = idx / (BM / LV);
			const int mrow = tile_row_m(L, g, tile, BM, row);
			lstm_e[gi] = mrow < g.M ? (unsigned) mrow + (unsigned) g.M * (unsigned) (bp.y * CB + cl) : 0xffffffffu;
			/* (every element of the array assigned: a partly initialised register array ends up in scratch memory) */
			lstm_forward_load_vec<T, LV>(E.lstm, lstm_e[gi] != 0xffffffffu ? lstm_e[gi] : 0u, lstm_in[gi]);
		}
	}

	/* --- table writer state: thread t < KC walks k = k0 + t, k0 + t + KC, ... from the first chunk's k0 --- */
	int tr, ts, tch;
	{
		const int k = chunk0 * KC + tid;
		tr = k % g.R;
		const int t = k / g.R;
		ts = t % g.S;
		tch = t / g.S;
	}
	const int eR = KC % g.R, eS = (KC / g.R) % g.S, eCh = (KC / g.R) / g.S;
	const int plane = g.NS * g.LH * g.LW;
	auto write_table = [&](int slot) {
		if (tid < KC) {
			const bool kv = tch < g.LC;
			const int dya = tr * g.RA, dyb = ts * g.RB;
			const int choff = kv ? plane * tch : 0;
			ktab[slot][tid] = make_int4(kv ? g.NS * (dya + g.LH * dyb) + choff : 0, kv ? dya : INVALID, dyb, choff);
			tr += eR;
			const int c1 = tr >= g.R;
			tr -= c1 ? g.R : 0;
			ts += eS + c1;
			const int c2 = ts >= g.S;
			ts -= c2 ? g.S : 0;
			tch += eCh + c2;
		}
	};

	/* --- per-thread gather state: a fixed group of VEC rows m --- */
	const int acol = tid % ACOLS, arow0 = tid / ACOLS;
	const int sb_shift = EPI == EPI_POOL ? L.sb_shift : 5;
	const int m = tile_row_m(L, g, tile, BM, acol * VEC, sb_shift);
	const bool mvalid = m < g.M;
	int n, ya0, yb0;
	{
		n = m % g.N;
		const int t = m / g.N;
		const int a = t % g.OA, b = t / g.OA;
		ya0 = a * g.SA + g.PA;
		yb0 = b * g.SB + g.PB;
	}
	const int base_m = n + g.NS * (ya0 + g.LH * yb0);      /* may be negative; only used when in range */
	const T* const zeros = reinterpret_cast<const T*>(g_zero_block);
	const T* bptr[BITER];
	#pragma unroll
	for (int it = 0; it < BITER; ++it) {
		const int idx = tid + it * THREADS;
		bptr[it] = wt + ((size_t) (chunk0 * KC + idx / BCOLS) * g.ldw + f0 + (idx % BCOLS) * VB);
	}
	const size_t bstep = (size_t) KC * g.ldw;

	/* With 16-byte loads and whole wavefronts per tile row, the A operand goes from global memory straight into
	 * LDS (lane i of a wavefront lands at the wavefront's LDS base + 16 i, whatever address it reads), which
	 * saves the registers, the LDS store instructions and the wait between load and store. Measured: 1-3 %
	 * faster in fp32, slower in fp64, so fp32 only. */
	constexpr bool DIRECT = sizeof(T) == 4 && VEC == 4 && ACOLS % 64 == 0 && PF == 1;
	const int arow_u = __builtin_amdgcn_readfirstlane(arow0);
	const int acol_u = __builtin_amdgcn_readfirstlane(acol / 64) * 64 * VEC;
	T areg[PF][DIRECT ? 1 : ASLOTS][VEC];
	T breg[PF][BITER][VB];

	/* `stage` (a std::integral_constant) names the register set of the chunk: chunk c uses set c % PF */
	auto load_tiles = [&](int slot, int abuf, auto stage) {
		constexpr int SG = decltype(stage)::value;
		#pragma unroll
		for (int s = 0; s < ASLOTS; ++s) {
			const int4 e = ktab[slot][arow0 + s * ARP];
			int ya = ya0 + e.y, yb = yb0 + e.z;
			int ok = mvalid;                 /* bitwise, not short-circuit: keep this branch-free */
			int off;
			if (DIVS) {
				const int qa = ya / g.DA, qb = yb / g.DB;
				ok &= (qa * g.DA == ya) & (qb * g.DB == yb);
				ya = qa;
				yb = qb;
				off = n + g.NS * (ya + g.LH * yb) + e.w;
			} else {
				off = base_m + e.x;
			}
			ok &= ((unsigned) ya < (unsigned) g.LH) & ((unsigned) yb < (unsigned) g.LW);
			const T* p = ok ? src + off : zeros;
			if constexpr (DIRECT)
				__builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*) p,
						(__attribute__((address_space(3))) void*) &As[abuf][arow_u + s * ARP][acol_u], 16, 0, 0);
			else
				vec_load_global<T, VEC>(areg[SG][s], p);
		}
		#pragma unroll
		for (int it = 0; it < BITER; ++it) {
			if (BVECS % THREADS == 0 || tid + it * THREADS < BVECS) {
				vec_load_global<T, VB>(breg[SG][it], bptr[it]);
				bptr[it] += bstep;
			}
		}
	};
	auto store_tiles = [&](int buf, auto stage) {
		constexpr int SG = decltype(stage)::value;
		if constexpr (!DIRECT) {
			#pragma unroll
			for (int s = 0; s < ASLOTS; ++s)
				vec_store<T, VEC>(&As[buf][arow0 + s * ARP][acol * VEC], areg[SG][s]);
		}
		#pragma unroll
		for (int it = 0; it < BITER; ++it) {
			const int idx = tid + it * THREADS;
			if (BVECS % THREADS == 0 || idx < BVECS) {
				const int brow = idx / BCOLS, bcol = idx % BCOLS;
				vec_store<T, VB>(&Bs[buf][brow][bcol * VB], breg[SG][it]);
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

	/* tables of chunks 0 .. PF, loads of chunks 0 .. PF - 1, chunk 0 into LDS */
	#pragma unroll
	for (int q = 0; q <= PF; ++q)
		write_table(q);
	__syncthreads();
	static_for<PF>([&](auto q) {
		if (decltype(q)::value < nchunks)
			load_tiles(decltype(q)::value, 0, q);
	});
	store_tiles(0, std::integral_constant<int, 0>());
	if constexpr (DIRECT)
		__builtin_amdgcn_s_waitcnt(0x0F70);  /* vmcnt(0): the direct loads have landed */
	__syncthreads();
	int slot_load = PF % NSLOT, slot_write = (PF + 1) % NSLOT;      /* table slots of chunk c + PF and c + PF + 1 */
	for (int c0 = 0; c0 < nchunks; c0 += PF)
	static_for<PF>([&](auto stage) {
		constexpr int SG = decltype(stage)::value;
		const int c = c0 + SG;
		if (c >= nchunks)
			return;                          /* the same for every thread of the block: no barrier is skipped by some */
		const int buf = c & 1;
		write_table(slot_write);
		if (c + PF < nchunks)
			load_tiles(slot_load, buf ^ 1, stage);      /* this chunk's registers went to LDS one chunk ago */
		slot_load = slot_load == NSLOT - 1 ? 0 : slot_load + 1;
		slot_write = slot_write == NSLOT - 1 ? 0 : slot_write + 1;
		constexpr std::integral_constant<int, (SG + 1) % PF> next_stage{};
		/* operand fragments are fetched one reduction step ahead of the MFMAs that use them */
		T xa[2][MB], wb[2][FB];
		vec_load<T, MB>(xa[0], &As[buf][lk][wm * WT_M + MB * lc]);
		vec_load<T, FB>(wb[0], &Bs[buf][lk][wf * WT_F + FB * lc]);
		#pragma unroll
		for (int st = 0; st < KC / KS; ++st) {
			const int cur = st & 1, nxt = cur ^ 1;
			if (st + 1 < KC / KS) {
				/* lgkmcnt(0): this step's operands, read one step ago, have landed. Waiting here, before the
				 * next step's reads go out, keeps the compiler from placing the same wait after them, where
				 * it would hold this step's MFMAs back until the reads just issued have returned as well. */
				__builtin_amdgcn_s_waitcnt(0xC07F);
				vec_load<T, MB>(xa[nxt], &As[buf][(st + 1) * KS + lk][wm * WT_M + MB * lc]);
				vec_load<T, FB>(wb[nxt], &Bs[buf][(st + 1) * KS + lk][wf * WT_F + FB * lc]);
			}
			/* the next chunk goes into the other LDS buffer ahead of the last step's MFMAs rather than after
			 * them: its stores (and the wait for its global loads) then overlap that MFMA work, and
			 * only the barrier itself remains between the chunks */
			if (KC / KS > 1 && st == KC / KS - 1 && c + 1 < nchunks)
				store_tiles(buf ^ 1, next_stage);
			/* issue order matters (a wave issues in order and stalls on a busy MFMA pipe): the LDS reads
			 * of the next step must go out before this step's MFMAs, so pin the schedule here */
			__builtin_amdgcn_sched_barrier(0);
			#pragma unroll
			for (int i = 0; i < FB; ++i)
				#pragma unroll
				for (int j = 0; j < MB; ++j)
					acc[i][j] = MF::mma(wb[cur][i], xa[cur][j], acc[i][j]);
			__builtin_amdgcn_sched_barrier(0);
		}
		if (KC / KS <= 1 && c + 1 < nchunks)
			store_tiles(buf ^ 1, next_stage);
		if constexpr (DIRECT)
			__builtin_amdgcn_s_waitcnt(0x0F70);  /* vmcnt(0): this wave's direct loads of the next chunk have landed */
		__syncthreads();
	});

	/* epilogue: D rows are filters (row rr of block i is filter FB*rr + i), D columns are m
	 * (column lc of block j is row MB*lc + j of the tile), so a lane owns MB adjacent outputs */
	constexpr int VS = MB * (int) sizeof(T) > 16 ? 16 / (int) sizeof(T) : MB;
	if (split) {
		/* partial sums of this part: a dense BF x BM tile (m fastest), always whole and aligned */
		T* ptile = partials + ((size_t) (local * bp.ny + bp.y) * L.ksplit + part) * (BM * BF);
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r) {
				T* dst = ptile + (size_t) (wf * WT_F + FB * acc_row<T>(r, lk) + i) * BM + wm * WT_M + MB * lc;
				#pragma unroll
				for (int j0 = 0; j0 < MB; j0 += VS) {
					T v[VS];
					#pragma unroll
					for (int j = 0; j < VS; ++j)
						v[j] = acc[i][j0 + j][r];
					vec_store<T, VS>(dst + j0, v);
				}
			}
		return;
	}
	if constexpr (EPI == EPI_LSTM) {
		/* The tile (bias added) goes through LDS so that the four gates of a state element, which lie in four column
		 * groups and so in different lanes and waves, meet in one thread; the tile's own buffer, not the operand
		 * buffers: only the short tiles have this epilogue, and theirs are too small for a whole tile. */
		constexpr int LROW = BM + 4;
		__shared__ __attribute__((aligned(16))) T lstm_stage[BF * LROW];
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r) {
				const int col = wf * WT_F + FB * acc_row<T>(r, lk) + i;
				const T bv = bias_s[col];
				T v[MB];
				#pragma unroll
				for (int j = 0; j < MB; ++j)
					v[j] = acc[i][j][r] + bv;
				T* dst = lstm_stage + col * LROW + wm * WT_M + MB * lc;
				#pragma unroll
				for (int j0 = 0; j0 < MB; j0 += VS)
					vec_store<T, VS>(dst + j0, *reinterpret_cast<T (*)[VS]>(&v[j0]));
			}
		__syncthreads();
		/* the arithmetic of all of a thread's elements before the first store: independent chains that the compiler
		 * may interleave (stores in between would keep them apart), which matters with a wavefront per SIMD */
		LstmForwardOutputs<T> res[LSTM_GROUPS][LV];
		T zh4[LSTM_GROUPS][LV][4];
		#pragma unroll
		for (int gi = 0; gi < LSTM_GROUPS; ++gi) {
			const int idx = tid + gi * THREADS, row = (idx % (BM / LV)) * LV, cl = idx / (BM / LV);
			#pragma unroll
			for (int gt = 0; gt < 4; ++gt) {
				T zv[LV];
				vec_load<T, LV>(zv, &lstm_stage[(gt * CB + cl) * LROW + row]);
				#pragma unroll
				for (int k = 0; k < LV; ++k)
					zh4[gi][k][gt] = zv[k];
			}
		}
		if (lstm_standard_acts(E.lstm.a)) {
			#pragma unroll
			for (int gi = 0; gi < LSTM_GROUPS; ++gi)
				#pragma unroll
				for (int k = 0; k < LV; ++k)
					res[gi][k] = lstm_forward_compute<T, true>(E.lstm, lstm_in[gi][k], true, zh4[gi][k]);
		} else {
			#pragma unroll
			for (int gi = 0; gi < LSTM_GROUPS; ++gi)
				#pragma unroll
				for (int k = 0; k < LV; ++k)
					res[gi][k] = lstm_forward_compute<T, false>(E.lstm, lstm_in[gi][k], true, zh4[gi][k]);
		}
		#pragma unroll
		for (int gi = 0; gi < LSTM_GROUPS; ++gi)
			if (lstm_e[gi] != 0xffffffffu)
				lstm_forward_store_vec<T, LV>(E.lstm, lstm_e[gi], res[gi]);
		return;
	}
	if constexpr (EPI == EPI_POOL) {
		/* Pre-activation values of a group of output columns go through LDS (the operand buffers are free now), so
		 * that the threads can be dealt out over (column, window, sample): a window's positions lie in different
		 * lanes and waves. A pass stages, for one accumulator block i, the RG accumulator rows of group q of every
		 * wave: FP = WAVES_F * RG columns x BM rows, as many as the buffers hold (every barrier between passes is a
		 * stall of the whole block). */
		constexpr int LROW = BM + 4, ROOM = 2 * KC * LDA / (WAVES_F * LROW), RG_MIN = std::is_same<T, float>::value ? 8 : 4;
		constexpr int RG = ROOM >= TL ? TL : ROOM >= TL / 2 ? TL / 2 : RG_MIN, GROUPS = TL / RG, FP = WAVES_F * RG;
		constexpr int REGS_PER_GROUP = MF::NACC / GROUPS;
		static_assert(FP * LROW <= 2 * KC * LDA, "the staging tile of the pooling epilogue reuses the A operand buffers");
		T* const stage = &As[0][0][0];
		const int SB = 1 << sb_shift, P = BM >> sb_shift, pa = P / L.pos_b;
		const int W = P / (E.prh * E.prw), wa_n = pa / E.prh;
		const int strip = tile / L.tile_rows, trow = tile - strip * L.tile_rows;
		const int ab = trow / L.sample_blocks, nb = trow - ab * L.sample_blocks;
		const int a_p0 = ab * wa_n, b_p0 = strip * (L.pos_b / E.prw);
		/* What an output's place asks of index arithmetic: the window's first value in a staged column, and the element
		 * offsets of column 0 in the pooled tensors, the arg-max cache and the full-size tensor. */
		struct Spot {
			int col;
			size_t pooled, ind, full;
		};
		const auto spot = [&](int s_i, int w) {
			const int wb = w / wa_n, wa = w - wb * wa_n;
			const int n = (nb << sb_shift) + s_i, a_p = a_p0 + wa, b_p = b_p0 + wb;
			return Spot { s_i + (((wa * E.prh) + pa * (wb * E.prw)) << sb_shift), (size_t) n + (size_t) g.N * (a_p + (size_t) E.OHp * b_p),
					((size_t) b_p * E.OHp + a_p) * ((size_t) g.F * g.N) + n,
					(size_t) n + (size_t) g.N * (a_p * E.prh + (size_t) g.OA * (b_p * E.prw)) };
		};
		/* The threads walk (samples, window, column), samples first and PV of them (one 16-byte access) per thread. When
		 * the windows of a pass divide the threads of a sample block evenly, a thread keeps its samples and window through
		 * every pass and only its column moves on. */
		constexpr int PV = VEC, PV_SHIFT = PV == 4 ? 2 : PV == 2 ? 1 : 0;
		const int sbv_shift = sb_shift - PV_SHIFT, SBV = 1 << sbv_shift;          /* the planner keeps SB >= PV */
		const int tps = THREADS >> sbv_shift, outputs = (FP * W * SBV + THREADS - 1) / THREADS;
		const bool fixed_spot = tps % W == 0;
		const int fl0 = (tid >> sbv_shift) / W, fl_step = tps / W;
		Spot sp = spot((tid & (SBV - 1)) << PV_SHIFT, (tid >> sbv_shift) % W);
		const int kstep = pa << sb_shift;
		const bool two_by_two = E.prh == 2 && E.prw == 2;
		const size_t pooled_plane = (size_t) g.N * E.OHp * E.OWp;
		act_dispatch(E.kind, [&](auto kc) {
			constexpr int KIND = decltype(kc)::value;
			#pragma unroll
			for (int i = 0; i < FB; ++i) {
				#pragma unroll
				for (int q = 0; q < GROUPS; ++q) {
					__syncthreads();
					#pragma unroll
					for (int r = 0; r < MF::NACC; ++r) {
						if (r / REGS_PER_GROUP != q)
							continue;
						const int arow = acc_row<T>(r, lk);
						const T bv = bias_s[wf * WT_F + FB * arow + i];
						T v[MB];
						#pragma unroll
						for (int j = 0; j < MB; ++j)
							v[j] = acc[i][j][r] + bv;
						T* dst = stage + (wf * RG + arow - RG * q) * LROW + wm * WT_M + MB * lc;
						#pragma unroll
						for (int j0 = 0; j0 < MB; j0 += VS)
							vec_store<T, VS>(dst + j0, *reinterpret_cast<T (*)[VS]>(&v[j0]));
					}
					__syncthreads();
					for (int pass = 0; pass < outputs; ++pass) {
						int fl;
						if (fixed_spot) {
							fl = fl0 + pass * fl_step;
							if (fl >= FP)
								break;
						} else {
							const int it = tid + pass * THREADS;
							if (it >= FP * W * SBV)
								break;
							const int t2 = it >> sbv_shift;
							fl = t2 / W;
							sp = spot((it & (SBV - 1)) << PV_SHIFT, t2 - fl * W);
						}
						const int f = f0 + (fl / RG) * WT_F + FB * (RG * q + fl % RG) + i;
						if (f >= g.F)
							continue;
						const T* col = stage + fl * LROW + sp.col;
						T zv[PV];
						if (E.pool_mean) {
							/* the mean of the window, summed width-major / height-minor as the layer of its own does
							 * (MeanPoolLayer.hpp:35-41); what the backward pass needs goes out at every position */
							T sum[PV];
							#pragma unroll
							for (int e = 0; e < PV; ++e)
								sum[e] = (T) 0;
							for (int k = 0; k < E.prw; ++k)
								for (int l = 0; l < E.prh; ++l) {
									vec_load<T, PV>(zv, col + k * kstep + l * SB);
									T y[PV];
									#pragma unroll
									for (int e = 0; e < PV; ++e) {
										y[e] = act_f_coded<T, KIND>(zv[e], E.p);
										sum[e] += y[e];
									}
									if (E.pre)
										vec_store_stream<T, PV>(E.pre + (sp.full + (size_t) g.N * (l + (size_t) g.OA * (k + (size_t) g.OB * f))),
												E.keep_input ? zv : y);
								}
							#pragma unroll
							for (int e = 0; e < PV; ++e)
								sum[e] = sum[e] / (T) (E.prh * E.prw);
							vec_store_stream<T, PV>(out + (sp.pooled + pooled_plane * f), sum);
							continue;
						}
						/* strict '>' from lowest(), width-major / height-minor scan (MaxPoolLayer.hpp:45-56) */
						T best[PV], best_pre[PV];
						unsigned bi[PV];
						vec_load<T, PV>(zv, col);
						#pragma unroll
						for (int e = 0; e < PV; ++e) {
							best[e] = std::numeric_limits<T>::lowest();
							best_pre[e] = zv[e];
							bi[e] = 0;
						}
						const auto consider = [&](const T (&z)[PV], unsigned at) {
							#pragma unroll
							for (int e = 0; e < PV; ++e) {
								const T y = act_f_coded<T, KIND>(z[e], E.p);
								if (y > best[e]) {
									best[e] = y;
									best_pre[e] = z[e];
									bi[e] = at;
								}
							}
						};
						if (two_by_two) {
							/* the usual window: its four positions fetched together, then scanned in the same order */
							T z1[PV], z2[PV], z3[PV];
							vec_load<T, PV>(z1, col + SB);
							vec_load<T, PV>(z2, col + kstep);
							vec_load<T, PV>(z3, col + kstep + SB);
							consider(zv, 0u);
							consider(z1, 1u);
							consider(z2, 2u);
							consider(z3, 3u);
						} else {
							for (int k = 0; k < E.prw; ++k)
								for (int l = 0; l < E.prh; ++l) {
									vec_load<T, PV>(zv, col + k * kstep + l * SB);
									consider(zv, (unsigned) (k * E.prh + l));
								}
						}
						vec_store_stream<T, PV>(out + (sp.pooled + pooled_plane * f), best);
						vec_store_stream<unsigned, PV>(E.inds + (sp.ind + (size_t) f * g.N), bi);
						if (E.pre)
							vec_store_stream<T, PV>(E.pre + (sp.pooled + pooled_plane * f), best_pre);
					}
				}
			}
		});
		return;
	}
	const bool vec_out = g.M % MB == 0 && (reinterpret_cast<uintptr_t>(out) & (VS * sizeof(T) - 1)) == 0;
	const int mm = tile_row_m(L, g, tile, BM, wm * WT_M + MB * lc);
	if constexpr (EPI == EPI_ACT) {
		act_dispatch(E.kind, [&](auto kc) {
			constexpr int KIND = decltype(kc)::value;
			#pragma unroll
			for (int i = 0; i < FB; ++i) {
				#pragma unroll
				for (int r = 0; r < MF::NACC; ++r) {
					const int f = f0 + wf * WT_F + FB * acc_row<T>(r, lk) + i;
					if (f >= g.F)
						continue;
					const T bv = bias_s[wf * WT_F + FB * acc_row<T>(r, lk) + i];
					const size_t o = (size_t) mm + (size_t) g.M * f;
					T z[MB], y[MB];
					#pragma unroll
					for (int j = 0; j < MB; ++j) {
						z[j] = acc[i][j][r] + bv;
						y[j] = act_f_coded<T, KIND>(z[j], E.p);
					}
					if (vec_out) {
						if (mm < g.M) {
							#pragma unroll
							for (int j0 = 0; j0 < MB; j0 += VS) {
								vec_store_stream<T, VS>(out + o + j0, *reinterpret_cast<T (*)[VS]>(&y[j0]));
								if (E.pre)
									vec_store_stream<T, VS>(E.pre + o + j0, *reinterpret_cast<T (*)[VS]>(&z[j0]));
							}
						}
					} else {
						#pragma unroll
						for (int j = 0; j < MB; ++j)
							if (mm + j < g.M) {
								out[o + j] = y[j];
								if (E.pre)
									E.pre[o + j] = z[j];
							}
					}
				}
			}
		});
		return;
	}
	if constexpr (EPI == EPI_STATS) {
		/* Moments of this tile's rows per output column, from the accumulators: per lane the sums of (z - c) and
		 * (z - c)^2 about a value c of the same column (the first row of the wave's rows: a shift from within the
		 * data, so the squares do not cancel), added over the lanes of a column by a butterfly, then the waves along
		 * m merged in ascending order by the update of Chan et al. */
		T* const red = &As[0][0][0];                    /* [WAVES_M][BF][4]: count, shift, sum, sum of squares */
		static_assert(WAVES_M * (WAVES_F * WT_F) * 4 <= 2 * KC * LDA, "the moment partials reuse the A operand buffers");
		/* The cross-lane sums stay inside the vector ALU (lane_group_sum), and the shift, one value per column from the
		 * first lane of each group, is read as a scalar (fp32; fp64 has few columns per lane and shuffles it). */
		T c[FB][MF::NACC], s1[FB][MF::NACC], s2[FB][MF::NACC];
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r)
				c[i][r] = acc[i][0][r] + bias_s[wf * WT_F + FB * acc_row<T>(r, lk) + i];
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r) {
				if constexpr (std::is_same<T, float>::value) {
					/* the first lane of each half of the wavefront, read as scalars */
					const int bits = __builtin_bit_cast(int, c[i][r]);
					const int lo = __builtin_amdgcn_readlane(bits, 0), hi = __builtin_amdgcn_readlane(bits, 32);
					c[i][r] = __builtin_bit_cast(float, lk == 0 ? lo : hi);
				} else {
					c[i][r] = __shfl(c[i][r], lane & ~(TL - 1), 64);
				}
			}
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r) {
				const T bv = bias_s[wf * WT_F + FB * acc_row<T>(r, lk) + i];
				s1[i][r] = (T) 0;
				s2[i][r] = (T) 0;
				#pragma unroll
				for (int j = 0; j < MB; ++j) {
					const T d = mm + j < g.M ? (acc[i][j][r] + bv) - c[i][r] : (T) 0;
					s1[i][r] += d;
					s2[i][r] += d * d;
				}
			}
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			#pragma unroll
			for (int r = 0; r < MF::NACC; ++r) {
				s1[i][r] = lane_group_sum<T, TL>(s1[i][r]);
				s2[i][r] = lane_group_sum<T, TL>(s2[i][r]);
			}
		/* rows of this wave that exist: all of them in the blocked order, else what is left of M */
		const int wave_rows = L.sample_blocks > 0 ? WT_M : max(0, min(WT_M, g.M - (tile * BM + wm * WT_M)));
		if (lc == TL - 1) {                  /* the lane that holds the group's totals */
			#pragma unroll
			for (int i = 0; i < FB; ++i)
				#pragma unroll
				for (int r = 0; r < MF::NACC; ++r) {
					T* dst = red + ((size_t) wm * BF + wf * WT_F + FB * acc_row<T>(r, lk) + i) * 4;
					dst[0] = (T) wave_rows;
					dst[1] = c[i][r];
					dst[2] = s1[i][r];
					dst[3] = s2[i][r];
				}
		}
		__syncthreads();
		for (int fl = tid; fl < BF; fl += THREADS) {
			if (f0 + fl >= g.F)
				continue;
			T n = (T) 0, mean = (T) 0, m2 = (T) 0;
			#pragma unroll
			for (int w = 0; w < WAVES_M; ++w) {
				const T* src4 = red + ((size_t) w * BF + fl) * 4;
				const T nb_ = src4[0];
				if (nb_ > (T) 0) {
					const T mb = src4[2] / nb_, meanb = src4[1] + mb, m2b = src4[3] - src4[2] * mb;
					const T nt = n + nb_, d = meanb - mean, wgt = nb_ / nt;
					mean += d * wgt;
					m2 += m2b + (d * d) * (n * wgt);
					n = nt;
				}
			}
			T* dst = E.stats + ((size_t) tile * g.F + (f0 + fl)) * 3;
			dst[0] = n;
			dst[1] = mean;
			dst[2] = m2;
		}
		/* the tile itself is stored below, like any other */
	}
	/* (the output map: plain except for the residue classes of a strided input gradient, which have no fused epilogue) */
	const size_t mm_out = EPI == EPI_NONE ? out_row(g, min(mm, g.M - 1)) : (size_t) mm;
	#pragma unroll
	for (int i = 0; i < FB; ++i) {
		#pragma unroll
		for (int r = 0; r < MF::NACC; ++r) {
			const int f = f0 + wf * WT_F + FB * acc_row<T>(r, lk) + i;
			if (f < g.F) {
				const T bv = bias_s[wf * WT_F + FB * acc_row<T>(r, lk) + i];
				T* dst = out + (mm_out + (size_t) g.out_M * f);
				if (vec_out) {
					if (mm < g.M) {
						#pragma unroll
						for (int j0 = 0; j0 < MB; j0 += VS) {
							T v[VS];
							#pragma unroll
							for (int j = 0; j < VS; ++j)
								v[j] = acc[i][j0 + j][r] + bv;
							vec_store_stream<T, VS>(dst + j0, v);
						}
					}
				} else {
					#pragma unroll
					for (int j = 0; j < MB; ++j)
						if (mm + j < g.M)
							dst[j] = acc[i][j][r] + bv;
				}
			}
		}
	}
}

/* How the weight-gradient launch is cut: tiles = ktiles * ftiles blocks per slice, `splits` slices. */
struct WgradSplit {
	int ktiles, tiles, splits, chunks_per_split, pixel_mode;
	int direct;     /* one slice only: the block adds its tile to the gradient itself, `partials` and `bias_partials` are the gradients */
};

/* ------------------------------------------------------------------------------------------------
 * Weight-gradient partials: P[k + K*f] = sum over this block's slice of m of A(m,k) * G(m,f), plus the
 * bias-gradient partials (column sums of G over the same slice) from the G tile already in LDS.
 * The reduction index m is the contiguous one, so both operand tiles are staged as [row][m] and a
 * lane fetches VR consecutive m with one 16-byte LDS read; since a sum may be taken in any order,
 * MFMA step e pairs reduction slot lk with m = mm + lk*VR + e for both operands.
 * The LDS tile is single-buffered: the global loads of the next chunk are in flight in registers
 * while the current chunk is multiplied, and two to three blocks per CU cover the barriers.
 * grid = tiles * splits blocks (1-D). Bias rows are dealt out over the k tiles (row f belongs to the
 * block with f % ktiles == k-tile index) so that every block does the same amount of extra work.
 * ---------------------------------------------------------------------------------------------- */
/* GMODE: where the G operand comes from. 0: `og` is it. 1 (WgradAct): og is the gradient behind a rectifier whose coded
 * outputs are act_y; the derivative is applied as a chunk goes into LDS, and the blocks of the first k tile write the
 * product to act_dz (if given). 2: og is the gradient behind a rectifier and a max pool whose windows tile the output
 * (2^pool_sh_a x 2^pool_sh_b, stride = receptor): og and act_y are pooled tensors, pool_inds the pool's arg-max cache in
 * the layout of MaxPoolLayer; an element of G is the pooled gradient times the derivative where the arg-max names its
 * position in the window and zero elsewhere, formed as the chunk goes into LDS - the full-size gradient is never
 * written (for layers whose input gradient nobody needs). */
template<typename T, int WAVES_K, int WAVES_F, int WT_K, int WT_F, int MC, int VEC, int GMODE>
__device__ __forceinline__ void wgrad_body(const T* __restrict__ src, const T* __restrict__ og, T* __restrict__ partials,
		T* __restrict__ bias_partials, const GatherGeom& g, const WgradSplit& plan, const T* __restrict__ act_y,
		T* __restrict__ act_dz, T act_p0, T act_p1, int bid, const unsigned* __restrict__ pool_inds = nullptr, int pool_sh_a = 0,
		int pool_sh_b = 0) {
	constexpr bool ACTG = GMODE != 0;
	/* (the activation's tensors as parameters of their own: pointers inside a structure are not known to point to global
	 * memory, and flat loads count against the LDS counter as well, see vec_load_global) */
	typedef Mfma<T> MF;
	constexpr int THREADS = 64 * WAVES_K * WAVES_F;
	constexpr int BK = WAVES_K * WT_K, BF = WAVES_F * WT_F;
	constexpr int VR = 16 / (int) sizeof(T);
	constexpr int LDM = MC + VR;
	constexpr int TL = MF::TL, KS = MF::KS;
	constexpr int KB = WT_K / TL, FB = WT_F / TL;
	constexpr int COLS = MC / VEC, RP = THREADS / COLS;
	constexpr int XSLOTS = (BK + RP - 1) / RP, GSLOTS = (BF + RP - 1) / RP;
	constexpr int Q = MC / VR;                               /* 16-byte groups per tile row */
	constexpr int BIAS_IT = (BF * Q + THREADS - 1) / THREADS;
	static_assert(THREADS % COLS == 0, "loader mapping");
	static_assert(MC % (VR * KS) == 0, "reduction chunk");
	static_assert(BK * LDM >= BF * Q, "bias reduction reuses the X tile");

	__shared__ __attribute__((aligned(16))) T Xs[BK][LDM];
	__shared__ __attribute__((aligned(16))) T Gs[BF][LDM];

	const int tid = threadIdx.x;
	/* blocks of one slice (its k and f tiles) get consecutive positions on one XCD: they read the same
	 * rows of G, which then come out of that XCD's L2 instead of HBM */
	const int pos = xcd_tile(bid, plan.tiles * plan.splits);
	if (pos >= plan.tiles * plan.splits)
		return;
	const int split = pos / plan.tiles, tile = pos - split * plan.tiles;
	const int ktiles = plan.ktiles;
	const int kt = tile % ktiles;
	const int k0 = kt * BK;
	const int f0 = (tile / ktiles) * BF;
	/* The slice of M. Pixel mode (N a multiple of MC): the slice is a range of output positions and is
	 * walked sample block by sample block (32 samples of every position, then the next 32), so the
	 * input rows that neighbouring positions share are reused while still in L2. Linear mode: a
	 * range of 32-row chunks of M in memory order. */
	const bool pixel_mode = plan.pixel_mode != 0;
	int chunk_count, pix0 = 0, npix = 1;
	if (pixel_mode) {
		const long positions = (long) g.OA * g.OB;
		pix0 = (int) (positions * split / plan.splits);
		npix = (int) (positions * (split + 1) / plan.splits) - pix0;
		chunk_count = npix * (g.N / MC);
	} else {
		const int total_chunks = (g.M + MC - 1) / MC;
		const int begin = split * plan.chunks_per_split;
		chunk_count = max(0, min(begin + plan.chunks_per_split, total_chunks) - begin);
	}

	const int col = tid % COLS, row0 = tid / COLS;
	/* The k rows a thread loads are the same in every chunk, so what the gather needs of them stays in registers
	 * instead of a table in LDS (whose reads sat in front of every global load): the displacements of the
	 * receptor position along both axes, packed as dya | dyb << 16 (both are below 32768, checked on the host;
	 * -1 for a row outside K or outside the tile), and the element offset that the row adds to the offset of
	 * the chunk's output position. */
	int krs[XSLOTS], koff[XSLOTS];
	#pragma unroll
	for (int s = 0; s < XSLOTS; ++s) {
		const int row = row0 + s * RP, k = k0 + row;
		const int r = k % g.R, t = k / g.R;
		const int sb = t % g.S, ch = t / g.S;
		const int dya = r * g.RA, dyb = sb * g.RB;
		krs[s] = (k < g.K && (BK % RP == 0 || row < BK)) ? (dya | dyb << 16) : -1;
		koff[s] = g.N * (dya + g.LH * dyb) + g.N * g.LH * g.LW * ch;
	}
	/* (n, a, b) of this thread's vector for the next chunk to load */
	int n, a, b, a0, b0, pleft = npix;
	if (pixel_mode) {
		n = col * VEC;
		a0 = a = pix0 % g.OA;
		b0 = b = pix0 / g.OA;
	} else {
		const int m = split * plan.chunks_per_split * MC + col * VEC;
		n = m % g.N;
		const int t = m / g.N;
		a0 = a = t % g.OA;
		b0 = b = t / g.OA;
	}
	const int eN = MC % g.N, eA = (MC / g.N) % g.OA, eB = (MC / g.N) / g.OA;

	T xreg[XSLOTS][VEC], greg[GSLOTS][VEC];
	/* ACTG: the activation outputs beside the gradient values, and where both came from; the derivative is applied
	 * when the chunk is stored to LDS, a chunk after its loads were issued, so that nothing waits for them here */
	T yreg[ACTG ? GSLOTS : 1][VEC];
	unsigned ireg[GMODE == 2 ? GSLOTS : 1][VEC];        /* GMODE 2: the windows' arg-max positions */
	unsigned pos_loaded = 0;                            /* ... and the position of the loaded rows in their window */
	int gm_loaded = 0;
	bool gvalid_loaded = false;

	auto load_tiles = [&]() {
		const int m = n + g.N * (a + g.OA * b);
		const bool mvalid = b < g.OB;
		const int ya0 = a * g.SA + g.PA, yb0 = b * g.SB + g.PB;
		const int base = n + g.N * (ya0 + g.LH * yb0);       /* may lie in the padding; only used when in range */
		#pragma unroll
		for (int s = 0; s < XSLOTS; ++s) {
			const int ya = ya0 + (krs[s] & 0xffff), yb = yb0 + (krs[s] >> 16);
			const bool ok = mvalid && krs[s] >= 0 && (unsigned) ya < (unsigned) g.LH && (unsigned) yb < (unsigned) g.LW;
			const int off = base + koff[s];
			if (ok) {
				vec_load<T, VEC>(xreg[s], src + off);
			} else {
				#pragma unroll
				for (int v = 0; v < VEC; ++v)
					xreg[s][v] = (T) 0;
			}
		}
		/* GMODE 2: the rows' window (ap, bp) of the pooled tensors, whose rows are mp = n + N (ap + OAp bp) */
		const int ap = a >> pool_sh_a, bp = b >> pool_sh_b, oap = g.OA >> pool_sh_a;
		const size_t mp = (size_t) n + (size_t) g.N * (ap + oap * bp), pooled_rows = (size_t) g.M >> (pool_sh_a + pool_sh_b);
		#pragma unroll
		for (int s = 0; s < GSLOTS; ++s) {
			const int row = row0 + s * RP;
			const int f = f0 + row;
			if (mvalid && f < g.F && (BF % RP == 0 || row < BF)) {
				if constexpr (GMODE == 2) {
					vec_load<T, VEC>(greg[s], og + (mp + pooled_rows * f));
					vec_load<T, VEC>(yreg[s], act_y + (mp + pooled_rows * f));
					vec_load<unsigned, VEC>(ireg[s], pool_inds + ((size_t) (bp * oap + ap) * ((size_t) g.F * g.N) + (size_t) f * g.N + n));
				} else {
					vec_load<T, VEC>(greg[s], og + ((size_t) m + (size_t) g.M * f));
					if constexpr (ACTG)
						vec_load<T, VEC>(yreg[s], act_y + ((size_t) m + (size_t) g.M * f));
				}
			} else {
				#pragma unroll
				for (int v = 0; v < VEC; ++v) {
					greg[s][v] = (T) 0;
					if constexpr (ACTG)
						yreg[s][v] = (T) 0;
					if constexpr (GMODE == 2)
						ireg[s][v] = 0xffffffffu;
				}
			}
		}
		if constexpr (GMODE == 2)
			pos_loaded = (unsigned) (((b - (bp << pool_sh_b)) << pool_sh_a) + (a - (ap << pool_sh_a)));
		gm_loaded = m;
		gvalid_loaded = mvalid;
		if (pixel_mode) {
			/* next position of the slice; after the last one, back to the first with the next samples */
			a += 1;
			const int c1 = a >= g.OA;
			a -= c1 ? g.OA : 0;
			b += c1;
			if (--pleft == 0) {
				pleft = npix;
				a = a0;
				b = b0;
				n += MC;
			}
		} else {
			/* advance m by MC with carries into (a, b) */
			n += eN;
			const int c1 = n >= g.N;
			n -= c1 ? g.N : 0;
			a += eA + c1;
			const int c2 = a >= g.OA;
			a -= c2 ? g.OA : 0;
			b += eB + c2;
		}
	};
	auto store_tiles = [&]() {
		#pragma unroll
		for (int s = 0; s < XSLOTS; ++s)
			if (BK % RP == 0 || row0 + s * RP < BK)
				vec_store<T, VEC>(&Xs[row0 + s * RP][col * VEC], xreg[s]);
		if constexpr (ACTG) {
			/* The rectifier family, without a branch on the kind (a switch here, even outside the loops, turned the
			 * register arrays into scratch memory): the derivative is 1 on the non-negative side and act_p0 + act_p1 * y
			 * on the negative side, which the coded output's sign bit names - 0 for ReLU, alpha for LeakyReLU,
			 * y + alpha for ELU, the expressions of act_b_coded. Rows outside the tile or the matrix were loaded as zeros. */
			#pragma unroll
			for (int s = 0; s < GSLOTS; ++s) {
				if (BF % RP == 0 || row0 + s * RP < BF) {
					const bool live = gvalid_loaded && f0 + row0 + s * RP < g.F;
					T dzv[VEC];
					#pragma unroll
					for (int v = 0; v < VEC; ++v) {
						const T slope = sign_bit(yreg[s][v]) ? act_p1 * yreg[s][v] + act_p0 : (T) 1;
						if constexpr (GMODE == 2)
							dzv[v] = live && ireg[s][v] == pos_loaded ? slope * greg[s][v] : (T) 0;
						else
							dzv[v] = live ? slope * greg[s][v] : (T) 0;
					}
					vec_store<T, VEC>(&Gs[row0 + s * RP][col * VEC], dzv);
					/* each element of G belongs to one (slice, f tile): the blocks of the first k tile write it */
					if (GMODE == 1 && act_dz != nullptr && kt == 0 && live)
						vec_store<T, VEC>(act_dz + ((size_t) gm_loaded + (size_t) g.M * (f0 + row0 + s * RP)), dzv);
				}
			}
		} else {
			#pragma unroll
			for (int s = 0; s < GSLOTS; ++s)
				if (BF % RP == 0 || row0 + s * RP < BF)
					vec_store<T, VEC>(&Gs[row0 + s * RP][col * VEC], greg[s]);
		}
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

	/* bias partial sums: item p = tid + it*THREADS covers 16-byte group p % Q of local row
	 * (p / Q) * ktiles + kt */
	T bacc[BIAS_IT];
	#pragma unroll
	for (int it = 0; it < BIAS_IT; ++it)
		bacc[it] = (T) 0;

	if (chunk_count > 0)
		load_tiles();
	for (int c = 0; c < chunk_count; ++c) {
		__syncthreads();              /* every wave is done reading the previous chunk */
		store_tiles();
		__syncthreads();
		if (c + 1 < chunk_count)
			load_tiles();
		/* operand fragments are fetched one group of VR reduction steps ahead of the MFMAs */
		T ga[2][FB][VR], xb[2][KB][VR];
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			vec_load<T, VR>(ga[0][i], &Gs[wf * WT_F + i * TL + lc][lk * VR]);
		#pragma unroll
		for (int j = 0; j < KB; ++j)
			vec_load<T, VR>(xb[0][j], &Xs[wk * WT_K + j * TL + lc][lk * VR]);
		#pragma unroll
		for (int st = 0; st < MC / (VR * KS); ++st) {
			const int cur = st & 1, nxt = cur ^ 1;
			if (st + 1 < MC / (VR * KS)) {
				const int mm = (st + 1) * VR * KS;
				#pragma unroll
				for (int i = 0; i < FB; ++i)
					vec_load<T, VR>(ga[nxt][i], &Gs[wf * WT_F + i * TL + lc][mm + lk * VR]);
				#pragma unroll
				for (int j = 0; j < KB; ++j)
					vec_load<T, VR>(xb[nxt][j], &Xs[wk * WT_K + j * TL + lc][mm + lk * VR]);
			}
			__builtin_amdgcn_sched_barrier(0);       /* next group's LDS reads go out before these MFMAs */
			#pragma unroll
			for (int e = 0; e < VR; ++e)
				#pragma unroll
				for (int i = 0; i < FB; ++i)
					#pragma unroll
					for (int j = 0; j < KB; ++j)
						acc[i][j] = MF::mma(ga[cur][i][e], xb[cur][j][e], acc[i][j]);
			__builtin_amdgcn_sched_barrier(0);
		}
		#pragma unroll
		for (int it = 0; it < BIAS_IT; ++it) {
			const int p = tid + it * THREADS;
			const int frow = (p / Q) * ktiles + kt;
			if (frow < BF) {
				T v[VR];
				vec_load<T, VR>(v, &Gs[frow][(p % Q) * VR]);
				#pragma unroll
				for (int e = 0; e < VR; ++e)
					bacc[it] += v[e];
			}
		}
	}

	const bool direct = plan.direct != 0;
	T* dst = partials + (size_t) split * ((size_t) g.K * g.F);
	if (direct) {
		/* gradients accumulate (StandardParameters.hpp:119): all of the tile's old values are fetched before the first
		 * is needed, so that the block waits for memory once and not once per value */
		#pragma unroll
		for (int i = 0; i < FB; ++i)
			#pragma unroll
			for (int j = 0; j < KB; ++j) {
				T old[MF::NACC];
				const int k = min(k0 + wk * WT_K + j * TL + lc, g.K - 1);
				#pragma unroll
				for (int r = 0; r < MF::NACC; ++r) {
					const int f = min(f0 + wf * WT_F + i * TL + acc_row<T>(r, lk), g.F - 1);
					old[r] = dst[(size_t) k + (size_t) g.K * f];
				}
				#pragma unroll
				for (int r = 0; r < MF::NACC; ++r)
					acc[i][j][r] += old[r];
			}
	}
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

	/* finish the bias partials: Q group sums per row, added in ascending group order */
	__syncthreads();
	T* bred = &Xs[0][0];
	#pragma unroll
	for (int it = 0; it < BIAS_IT; ++it) {
		const int p = tid + it * THREADS;
		const int frow = (p / Q) * ktiles + kt;
		if (frow < BF)
			bred[frow * Q + p % Q] = bacc[it];
	}
	__syncthreads();
	if (tid < BF && tid % ktiles == kt && f0 + tid < g.F && bias_partials != nullptr) {
		T s = (T) 0;
		#pragma unroll
		for (int q = 0; q < Q; ++q)
			s += bred[tid * Q + q];
		T* o = bias_partials + ((size_t) split * g.F + f0 + tid);
		*o = direct ? *o + s : s;
	}
}

template<typename T, int WAVES_K, int WAVES_F, int WT_K, int WT_F, int MC, int VEC, int MIN_WAVES, bool ACTG = false>
__global__ __launch_bounds__(64 * WAVES_K * WAVES_F, MIN_WAVES)      /* MIN_WAVES: wavefronts per SIMD the registers must allow */
void wgrad_kernel(const T* __restrict__ src, const T* __restrict__ og, T* __restrict__ partials,
		T* __restrict__ bias_partials, const GatherGeom g, const WgradSplit plan, const T* __restrict__ act_y,
		T* __restrict__ act_dz, T act_p0, T act_p1) {
	wgrad_body<T, WAVES_K, WAVES_F, WT_K, WT_F, MC, VEC, ACTG ? 1 : 0>(src, og, partials, bias_partials, g, plan, act_y, act_dz, act_p0, act_p1,
			(int) blockIdx.x);
}

/* The weight gradient of a layer behind a rectifier and a max pool, from the pooled gradient (wgrad_body, GMODE 2). */
template<typename T, int WAVES_K, int WAVES_F, int WT_K, int WT_F, int MC, int VEC>
__global__ __launch_bounds__(64 * WAVES_K * WAVES_F)
void wgrad_pooled_kernel(const T* __restrict__ src, const T* __restrict__ og, T* __restrict__ partials,
		T* __restrict__ bias_partials, const GatherGeom g, const WgradSplit plan, const T* __restrict__ act_y, T act_p0, T act_p1,
		const unsigned* __restrict__ pool_inds, int pool_sh_a, int pool_sh_b) {
	wgrad_body<T, WAVES_K, WAVES_F, WT_K, WT_F, MC, VEC, 2>(src, og, partials, bias_partials, g, plan, act_y, (T*) nullptr, act_p0, act_p1,
			(int) blockIdx.x, pool_inds, pool_sh_a, pool_sh_b);
}

/* A layer's input gradient and its weight gradient in one launch, for layers whose two launches are a few microseconds
 * each and wait for nothing but the same upstream gradient (the last layers of a network: a dependent launch costs 4-5 us
 * however little it does). The gather GEMM's blocks keep their places (x below gather_x); the weight gradient's blocks,
 * one wavefront each (the 32 x 32 tile), are the blocks with x from gather_x on, numbered row by row of the grid. */
template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int VEC>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_F)
void gather_with_wgrad_kernel(const T* __restrict__ src, const T* __restrict__ wt, T* __restrict__ out, const GatherGeom g,
		const GatherLaunch L, int gather_x, const T* __restrict__ w_src, const T* __restrict__ w_og, T* __restrict__ w_partials,
		T* __restrict__ w_bias_partials, const GatherGeom w_g, const WgradSplit w_plan) {
	if ((int) blockIdx.x < gather_x) {
		const Epilogue<T> none = { 0, (T) 0, nullptr, nullptr, 1, 1, 1, 1, nullptr, {} };
		gather_gemm_body<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_NONE, 1>(src, wt, (const T*) nullptr, out, g, L, (T*) nullptr, none,
				BlockPlace{ (int) blockIdx.x, (int) blockIdx.y, (int) gridDim.y });
	} else {
		if (threadIdx.x >= 64)
			return;
		const int bid = ((int) blockIdx.x - gather_x) + ((int) gridDim.x - gather_x) * (int) blockIdx.y;
		if (bid >= (w_plan.tiles * w_plan.splits + 7) / 8 * 8)
			return;
		wgrad_body<T, 1, 1, 32, 32, 32, VEC, 0>(w_src, w_og, w_partials, w_bias_partials, w_g, w_plan,
				(const T*) nullptr, (T*) nullptr, (T) 0, (T) 0, bid);
	}
}

/* dst[i] += sum_s partials[s][i] for 64 outputs of one matrix: block `blk` of it covers outputs [64 blk, 64 blk + 64)
 * with GR groups of threads, V consecutive outputs per thread; group j adds the partials s = j, j+GR, j+2GR, ... in
 * ascending order and the group sums are then added in ascending order, so the summation order is fixed and results
 * are reproducible. For V > 1 the count is a multiple of V and the partials are 16-byte aligned. */
template<typename T, int V>
__device__ __forceinline__ void reduce_partials_block(const T* __restrict__ partials, T* __restrict__ dst, size_t count, int blk,
		int splits, T (&lds)[16][64]) {
	constexpr int OV = 64 / V, GR = 256 / OV;
	static_assert(GR <= 16, "group sums fit the staging array");
	const int ox = (threadIdx.x % OV) * V, grp = threadIdx.x / OV;
	const size_t i = (size_t) blk * 64 + ox;
	T s[V];
	#pragma unroll
	for (int e = 0; e < V; ++e)
		s[e] = (T) 0;
	if (i < count)
		for (int p = grp; p < splits; p += GR) {
			T v[V];
			vec_load<T, V>(v, partials + (size_t) p * count + i);
			#pragma unroll
			for (int e = 0; e < V; ++e)
				s[e] += v[e];
		}
	#pragma unroll
	for (int e = 0; e < V; ++e)
		lds[grp][ox + e] = s[e];
	__syncthreads();
	const size_t o = (size_t) blk * 64 + threadIdx.x;
	if (threadIdx.x < 64 && o < count) {
		T total = lds[0][threadIdx.x];
		#pragma unroll
		for (int j = 1; j < GR; ++j)
			total += lds[j][threadIdx.x];
		dst[o] += total;
	}
}

/* The same sums for a small gradient (a few thousand values) cut into many partials: a wavefront per output (four per
 * block), lane l adds the partials s = l, l + 64, ... in ascending order and the 64 lane sums are combined by a fixed
 * shuffle tree. With few outputs the form above is a handful of blocks walking hundreds of partials one after the other. */
template<typename T>
__device__ __forceinline__ void reduce_partials_wide_block(const T* __restrict__ partials, T* __restrict__ dst, size_t count, int blk,
		int splits) {
	/* Neighbouring outputs share the cache lines of every slice: the blocks of one XCD take a contiguous range of outputs,
	 * so that a line is fetched by one L2, not by all eight (the entry's blocks start at a multiple of 8 and are a
	 * multiple of 8, see reduce_partials_many). */
	blk = xcd_tile(blk, (int) (((count + 3) / 4 + 7) / 8 * 8));
	const size_t i = (size_t) blk * 4 + threadIdx.x / 64;
	if (i >= count)
		return;
	const int lane = threadIdx.x % 64;
	T s = (T) 0;
	/* eight slices' loads are issued before the first of their additions (one after the other they are a chain of memory
	 * round trips); the additions keep their order */
	constexpr int AHEAD = 8;
	for (int p0 = lane; p0 < splits; p0 += 64 * AHEAD) {
		T v[AHEAD];
		#pragma unroll
		for (int j = 0; j < AHEAD; ++j) {
			const int p = p0 + 64 * j;
			v[j] = p < splits ? partials[(size_t) p * count + i] : (T) 0;
		}
		#pragma unroll
		for (int j = 0; j < AHEAD; ++j)
			if (p0 + 64 * j < splits)
				s += v[j];
	}
	#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		s += __shfl_down(s, off, 64);
	if (lane == 0)
		dst[i] += s;
}

/* The partial sums of up to REDUCE_BATCH matrices (the weight and the bias gradients of several layers) added to their
 * gradients in one launch: block b belongs to the entry whose range of blocks holds it. Every entry is summed in the
 * order the forms above fix, whatever else shares the launch. */
template<typename T>
__global__ __launch_bounds__(256)
void reduce_partials_many_kernel(const ReduceBatch<T> batch) {
	__shared__ T lds[16][64];
	int e = 0;
	while (e + 1 < batch.count && (int) blockIdx.x >= batch.e[e + 1].first_block)
		++e;
	const ReduceEntry<T>& q = batch.e[e];
	const int blk = (int) blockIdx.x - q.first_block;
	if (q.wide)
		reduce_partials_wide_block<T>(q.partials, q.dst, q.count, blk, q.splits);
	else if (q.vec)
		reduce_partials_block<T, 16 / (int) sizeof(T)>(q.partials, q.dst, q.count, blk, q.splits, lds);
	else
		reduce_partials_block<T, 1>(q.partials, q.dst, q.count, blk, q.splits, lds);
}

/* Forward weights: wt[k][f] = w[k + K*f], zero-padded to Kp rows x ldw columns. gate_block > 0: the columns in the
 * order of lstm_gate_column (F = 4 * hidden). */
template<typename T>
__global__ void prep_fwd_weights_kernel(const T* __restrict__ w, T* __restrict__ wt, int K, int F, int Kp, int ldw,
		int gate_block = 0) {
	const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= (size_t) Kp * ldw)
		return;
	const int f = (int) (i % ldw), k = (int) (i / ldw);
	const int fs = gate_block > 0 && f < F ? lstm_gate_column(f, gate_block, F / 4) : f;
	wt[i] = (k < K && f < F) ? w[(size_t) k + (size_t) K * fs] : (T) 0;
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

/* Input-gradient weights of one residue class of a strided convolution (see StridedClasses): the receptor rows
 * r0, r0 + sv, ... and columns s0, s0 + sh, ... only, wt[k' = r' + Rc*(s' + Sc*f)][c] = w[(r0 + sv r') + RH*((s0 + sh s') + RW*c) + K*f]. */
template<typename T>
__global__ void prep_dgrad_class_weights_kernel(const T* __restrict__ w, T* __restrict__ wt, int RH, int RW, int C, int F,
		int r0, int sv, int Rc, int s0, int sh, int Sc, int Kp, int ldw) {
	const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= (size_t) Kp * ldw)
		return;
	const int c = (int) (i % ldw), kp = (int) (i / ldw);
	const int taps = Rc * Sc;
	const int tap = kp % taps, f = kp / taps;
	const int r = r0 + sv * (tap % Rc), sb = s0 + sh * (tap / Rc);
	wt[i] = (f < F && c < C) ? w[(size_t) (r + RH * (sb + RW * c)) + (size_t) (RH * RW * C) * f] : (T) 0;
}

int round_up(int v, int to) {
	return (v + to - 1) / to * to;
}

constexpr int WT_ROW_PAD = 64;     /* a multiple of every KC: the last reduction chunk reads whole chunks of weight rows */
constexpr int WT_COL_PAD = 128;    /* >= every BF */
/* Compute units and LDS bytes per compute unit of the current device, from the runtime (256 and 160 KB on an MI355X;
 * a partitioned device reports its share), asked once. */
struct DeviceShape {
	int cus, lds_per_cu;
	DeviceShape() {
		int dev = 0;
		hipDeviceProp_t prop;
		CATTLE_HIP_CHECK(hipGetDevice(&dev));
		CATTLE_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
		cus = std::max(1, prop.multiProcessorCount);
		lds_per_cu = (int) std::max<size_t>(64 * 1024, prop.maxSharedMemoryPerMultiProcessor);
	}
};
const DeviceShape& device_shape() {
	static const DeviceShape shape;
	return shape;
}


/* Grow-only device scratch for split reductions. Calls into the library are serialised and issued on
 * one stream, so a later call may reuse (or, after hipFree's implicit synchronisation, replace) it. */
void* split_workspace(size_t bytes) {
	static void* ptr = nullptr;
	static size_t cap = 0;
	static uint64_t born = 0;
	if (bytes > cap) {
		forbid_while_capturing("growing the scratch buffer of the split reductions (run the step once before recording it)");
		/* every layer shares this buffer: a living graph recorded since it was allocated may point into it */
		if (ptr && pinned_by_graph(born))
			throw Error(ERR_STATE, "a recorded graph may point into the scratch buffer of the split reductions, which this call "
					"has to grow: destroy the graph (cattle_hip_graph_destroy) first, or run this problem once before recording");
		if (ptr)
			(void) hipFree(ptr);
		ptr = nullptr;
		cap = 0;
		const size_t want = (bytes + 4095) / 4096 * 4096;
		CATTLE_HIP_CHECK(hipMalloc(&ptr, want));
		cap = want;
		born = alloc_clock_tick();
	}
	return ptr;
}

/* Where a launch that must not allocate takes its scratch memory from: a caller-provided range of device memory that
 * is handed out front to back. A null arena means the library's own grow-only buffers. */
struct ScratchArena {
	char* base;
	size_t cap, used;
	void* take(size_t bytes, const char* what) {
		const size_t at = (used + 255) / 256 * 256;
		if (at + bytes > cap)
			throw Error(ERR_INVALID, std::string("the ") + what + " of this problem (" + std::to_string(bytes) +
					" bytes) do not fit the static scratch buffer of " + std::to_string(cap) + " bytes");
		used = at + bytes;
		return base + at;
	}
};

/* The scratch memory of the entry point that allocates nothing: a fixed array in the code object, so it exists once
 * per device for the life of the process and no call ever allocates or frees it. Its name is only a stand-in on the
 * host; the device address comes from hipGetSymbolAddress, once per device, and is what kernels and copies are given. */
constexpr size_t STATIC_SCRATCH_BYTES = (size_t) 72 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
void* g_scratch_ptr[MAX_DEVICES] = { nullptr };

/* ------------------------------------------------------------------------------------------------
 * The same gathered GEMM, out[M x F] = gather(src)[M x K] * wt[K x F] (+ bias), for F <= 4 output columns (NC = 8: five to
 * eight, unstrided problems with 16-byte accesses: at 8 columns the vector ALU still beats 32-column matrix tiles that
 * are three quarters padding, 81 -> 61 us on an 81,920 x 1152 x 8 input gradient; eight waves per block sharing the
 * reduction instead of four were slower on every problem tried): the input
 * gradient of a network's first convolution (its columns are the image's channels), a transposed convolution that
 * ends in one or three channels, a convolution with a handful of filters. On 32 x 32 matrix tiles such a problem is
 * seven eighths padding (measured on a 3 x 3 x 32 -> 3 input gradient: the matrix pipes busy half of the kernel's
 * time with zeros) and a strided one keeps all taps in the reduction although only 1 / (sv sh) of them reach a
 * given output. Here a lane owns VEC consecutive rows m (consecutive samples of one output position), reads their
 * operand values straight from global memory, coalesced along the sample index, and multiplies each with the F
 * weights of its reduction row, which are wave-uniform (scalar loads): no LDS staging, no padding, and a tap that
 * does not reach the lane's position (zero padding, or a stride that does not divide) costs a predicate. The
 * source channels are dealt over the four waves of a block, whose sums meet in LDS and are added in ascending
 * wave order: the summation order depends on the geometry only.
 * ---------------------------------------------------------------------------------------------- */
constexpr int FEW_COLUMNS = 4, SOME_COLUMNS = 8;
template<typename T, int VEC, bool DIVS, int UNROLL, int NC = FEW_COLUMNS>
__device__ __forceinline__ void few_columns_body(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias,
		T* __restrict__ out, const GatherGeom& g, int block, int act_kind = -1, T act_p = (T) 0, T* __restrict__ act_pre = nullptr) {
	constexpr int WAVES = 4, ROWS = 64 * VEC;
	const int lane = threadIdx.x % 64;
	const int wave = __builtin_amdgcn_readfirstlane((int) threadIdx.x / 64);
	/* The block's rows: 64 VEC consecutive m (samples of one output position, mostly), or - unstrided problems whose batch is
	 * a multiple of 32 and whose output divides into patches - 32 samples of a patch of 2 x (64 VEC / 64) positions: the
	 * taps of neighbouring positions read the same source rows, so a block of a patch touches a third of the source
	 * bytes that a block of one position's samples does, and the rest comes out of the caches (a 3 x 3 x 64 -> 3
	 * convolution over 262,144 rows fetched its 67 MB source six times over). */
	constexpr int LPS = 32 / VEC, PATCH_A = 2, PATCH_B = 64 / LPS / PATCH_A;
	/* (where fetches rather than arithmetic bound the kernel: up to four columns, and a source that the L2 caches
	 * together do not hold - with eight columns, or a source of 17 and 42 MB, patches were 10-14 % slower: their loads
	 * are 128-byte pieces where the other order reads a kilobyte at a stretch) */
	const bool patches = !DIVS && VEC > 1 && NC <= FEW_COLUMNS && g.N % 32 == 0 && g.OA % PATCH_A == 0 && g.OB % PATCH_B == 0 &&
			(size_t) g.NS * g.LH * g.LW * g.LC * sizeof(T) > ((size_t) 48 << 20);
	int m, n, ya0, yb0;
	bool mvalid;
	if (patches) {
		const int sbs = g.N / 32, pas = g.OA / PATCH_A;
		const int patch = block / sbs, pb_i = patch / pas, pos = lane / LPS;
		const int a = (patch - pb_i * pas) * PATCH_A + pos % PATCH_A, b = pb_i * PATCH_B + pos / PATCH_A;
		n = (block - patch * sbs) * 32 + (lane % LPS) * VEC;
		m = n + g.N * (a + g.OA * b);
		mvalid = b < g.OB;                       /* (blocks past the last one: the grid is rounded up) */
		ya0 = a * g.SA + g.PA;
		yb0 = b * g.SB + g.PB;
	} else {
		m = block * ROWS + lane * VEC;
		mvalid = m < g.M;                        /* whole vectors: M is a multiple of VEC */
		n = m % g.N;
		const int t = m / g.N;
		const int a = t % g.OA, b = t / g.OA;
		ya0 = a * g.SA + g.PA;
		yb0 = b * g.SB + g.PB;
	}
	constexpr int LOADS_IN_FLIGHT = UNROLL > 0 ? UNROLL : 1;
	constexpr int WL = NC == 3 ? 4 : NC;     /* a reduction row's weights are loaded as one, two, four or eight values */
	const int plane = g.NS * g.LH * g.LW;
	const int taps = g.R * g.S;
	T acc[NC][VEC];
	#pragma unroll
	for (int c = 0; c < NC; ++c)
		#pragma unroll
		for (int i = 0; i < VEC; ++i)
			acc[c][i] = (T) 0;
	if constexpr (UNROLL == 0) {
		/* Few source channels (a first layer's forward pass, a transposed convolution that ends in an image): the loop over
		 * taps below would wait for memory once per tap with a load or two in flight. Here the reduction steps (tap-major,
		 * channels within a tap) are dealt over the waves in contiguous shares and a wave takes its share in batches whose
		 * loads are all in flight together: a step that does not reach a row (zero padding) or lies past the share reads a
		 * block of zeros instead of branching. The address arithmetic is paid per step, not per tap: with many channels
		 * per tap the loop below is the faster one (4 x 4 x 3 -> 3 on 25,600 rows 6.9 -> 4.7 us; 3 x 3 x 32 -> 3 on 131,072
		 * rows 14.7 -> 22.7 us). */
		constexpr int BATCH = sizeof(T) == 4 ? 12 : 8;
		const int total = taps * g.LC, per = (total + WAVES - 1) / WAVES;
		const int s0 = wave * per, s1 = min(total, s0 + per);
		int tap = s0 / g.LC, ch = s0 - tap * g.LC;
		int sb = tap / g.R, r = tap - sb * g.R;
		const T* const zeros = reinterpret_cast<const T*>(g_zero_block);
		const int base = n + g.NS * (ya0 + g.LH * yb0);
		for (int s = s0; s < s1; s += BATCH) {
			T v[BATCH][VEC], wk[BATCH][WL];
			#pragma unroll
			for (int j = 0; j < BATCH; ++j) {
				const bool live = s + j < s1;        /* wave-uniform */
				const int da = r * g.RA, db = sb * g.RB;
				const bool ok = mvalid && live && (unsigned) (ya0 + da) < (unsigned) g.LH && (unsigned) (yb0 + db) < (unsigned) g.LW;
				vec_load_global<T, VEC>(v[j], ok ? src + (base + g.NS * (da + g.LH * db) + plane * ch) : zeros);
				/* reduction row k = r + R (s + S ch); the prepared weights hold its F values (zero-padded) first in its row */
				vec_load_global<T, WL>(wk[j], wt + (size_t) (live ? r + g.R * (sb + g.S * ch) : 0) * g.ldw);
				if (!live) {
					#pragma unroll
					for (int c = 0; c < NC; ++c)
						wk[j][c] = (T) 0;
				}
				const bool last_ch = ch + 1 == g.LC, last_r = r + 1 == g.R;
				ch = last_ch ? 0 : ch + 1;
				sb += last_ch && last_r ? 1 : 0;
				r = last_ch ? (last_r ? 0 : r + 1) : r;
			}
			#pragma unroll
			for (int j = 0; j < BATCH; ++j)
				#pragma unroll
				for (int c = 0; c < NC; ++c)
					#pragma unroll
					for (int i = 0; i < VEC; ++i)
						acc[c][i] += v[j][i] * wk[j][c];
		}
	} else {
		/* the source channels are dealt over the waves; a tap that reaches none of a wavefront's rows (zero padding, or a
		 * stride that does not divide: its rows share an output position or a few) is skipped whole */
		const int per = (g.LC + WAVES - 1) / WAVES;
		const int w0 = wave * per, w1 = min(g.LC, w0 + per);
		/* With patches, whole batches of channels outermost and the taps inside: what a tap's loads bring into the caches
		 * is what the next taps of the same channels read at the neighbouring positions, a few kilobytes later instead
		 * of after all of the wave's channels. Otherwise (and for a share that is not whole batches) tap by tap over all
		 * of the wave's channels: the per-tap arithmetic once. */
		const int group = patches && per % LOADS_IN_FLIGHT == 0 ? LOADS_IN_FLIGHT : max(per, 1);
		for (int c0 = w0; c0 < w1; c0 += group) {
		const int c1 = min(w1, c0 + group);
		for (int sb = 0; sb < g.S; ++sb)
			for (int r = 0; r < g.R; ++r) {
				int ya = ya0 + r * g.RA, yb = yb0 + sb * g.RB;
				bool ok = mvalid;
				if (DIVS) {
					const int qa = ya / g.DA, qb = yb / g.DB;
					ok = ok && qa * g.DA == ya && qb * g.DB == yb;
					ya = qa;
					yb = qb;
				}
				ok = ok && (unsigned) ya < (unsigned) g.LH && (unsigned) yb < (unsigned) g.LW;
				if (__builtin_amdgcn_ballot_w64(ok) == 0)
					continue;
				const T* p = src + (ok ? n + g.NS * (ya + g.LH * yb) + plane * c0 : 0);
				/* reduction row k = r + R (s + S ch); the prepared weights hold its F values (zero-padded) first in its row */
				const T* w = wt + (size_t) (r + g.R * (sb + g.S * c0)) * g.ldw;
				const size_t wstep = (size_t) taps * g.ldw;
				/* UNROLL loads in flight per wait; what is left over of a wave's channels goes one load at a time */
				#pragma unroll LOADS_IN_FLIGHT
				for (int ch = c0; ch < c1; ++ch) {
					T v[VEC];
					if (ok) {
						vec_load_global<T, VEC>(v, p);
					} else {
						#pragma unroll
						for (int i = 0; i < VEC; ++i)
							v[i] = (T) 0;
					}
					T wk[WL];
					vec_load_global<T, WL>(wk, w);
					#pragma unroll
					for (int c = 0; c < NC; ++c)
						#pragma unroll
						for (int i = 0; i < VEC; ++i)
							acc[c][i] += v[i] * wk[c];
					p += ok ? plane : 0;
					w += wstep;
				}
			}
		}
	}
	__shared__ T red[WAVES - 1][NC][ROWS];
	if (wave > 0) {
		#pragma unroll
		for (int c = 0; c < NC; ++c)
			vec_store<T, VEC>(&red[wave - 1][c][lane * VEC], acc[c]);
	}
	__syncthreads();
	if (wave == 0 && mvalid) {
		#pragma unroll
		for (int c = 0; c < NC; ++c) {
			if (c < g.F) {
				#pragma unroll
				for (int q = 0; q < WAVES - 1; ++q) {
					T part[VEC];
					vec_load<T, VEC>(part, &red[q][c][lane * VEC]);
					#pragma unroll
					for (int i = 0; i < VEC; ++i)
						acc[c][i] += part[i];
				}
				const T bv = bias ? bias[c] : (T) 0;
				#pragma unroll
				for (int i = 0; i < VEC; ++i)
					acc[c][i] += bv;
				if (act_kind < 0)
					vec_store<T, VEC>(out + (out_row(g, m) + (size_t) g.out_M * c), acc[c]);
			}
		}
		/* an element-wise activation on the way out (the fused forward pass of a kernel layer and its activation: coded
		 * outputs, and the inputs too where the backward pass needs them; 16-byte accesses, plain output map) */
		if (act_kind >= 0)
			act_dispatch(act_kind, [&](auto kc) {
				#pragma unroll
				for (int c = 0; c < NC; ++c)
					if (c < g.F) {
						T y[VEC];
						#pragma unroll
						for (int i = 0; i < VEC; ++i)
							y[i] = act_f_coded<T, decltype(kc)::value>(acc[c][i], act_p);
						const size_t o = (size_t) m + (size_t) g.M * c;
						vec_store_stream<T, VEC>(out + o, y);
						if (act_pre)
							vec_store_stream<T, VEC>(act_pre + o, acc[c]);
					}
			});
	}
}

/* Which 64 VEC rows block `bid` of a grid of (blocks rounded up to eight) takes: every XCD a contiguous range of the rows,
 * so that the blocks of neighbouring output positions, which read the same source rows through different taps, share an
 * L2 (dealt round-robin, an 81,920 x 1152 x 8 input gradient fetched its 42 MB source eight times over: 349 MB). */
template<int VEC>
__device__ __forceinline__ int few_columns_block(const GatherGeom& g, int bid) {
	return xcd_tile(bid, (g.M + 64 * VEC - 1) / (64 * VEC));
}

template<typename T, int VEC, bool DIVS, int UNROLL>
__global__ __launch_bounds__(256)
void few_columns_gather_kernel(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias,
		T* __restrict__ out, const GatherGeom g) {
	few_columns_body<T, VEC, DIVS, UNROLL>(src, wt, bias, out, g, few_columns_block<VEC>(g, (int) blockIdx.x));
}

template<typename T, int VEC, int UNROLL, int NC = FEW_COLUMNS>
__global__ __launch_bounds__(256)
void few_columns_plain_kernel(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias,
		T* __restrict__ out, const GatherGeom g, int act_kind, T act_p, T* __restrict__ act_pre) {
	few_columns_body<T, VEC, false, UNROLL, NC>(src, wt, bias, out, g, few_columns_block<VEC>(g, (int) blockIdx.x), act_kind, act_p, act_pre);
}

/* An input gradient of a few columns and the layer's weight gradient in one launch (see gather_with_wgrad_kernel: both
 * wait for the same upstream gradient only, and a dependent launch costs 4-5 us however little it does): blocks below
 * gather_blocks form the input gradient, the others are the weight gradient's one-wavefront blocks. */
template<typename T, int VEC, int UNROLL, int NC>
__global__ __launch_bounds__(256)
void few_columns_with_wgrad_kernel(const T* __restrict__ src, const T* __restrict__ wt, T* __restrict__ out, const GatherGeom g,
		int gather_blocks, const T* __restrict__ w_src, const T* __restrict__ w_og, T* __restrict__ w_partials,
		T* __restrict__ w_bias_partials, const GatherGeom w_g, const WgradSplit w_plan) {
	if ((int) blockIdx.x < gather_blocks) {
		few_columns_body<T, VEC, false, UNROLL, NC>(src, wt, (const T*) nullptr, out, g, few_columns_block<VEC>(g, (int) blockIdx.x));
	} else {
		if (threadIdx.x >= 64)
			return;
		wgrad_body<T, 1, 1, 32, 32, 32, VEC, 0>(w_src, w_og, w_partials, w_bias_partials, w_g, w_plan,
				(const T*) nullptr, (T*) nullptr, (T) 0, (T) 0, (int) blockIdx.x - gather_blocks);
	}
}

/* ------------------------------------------------------------------------------------------------
 * The weight gradient of a convolution with up to four filters (the last layer of an image decoder: many channels in, an
 * image out), dW[K x F] = patches(x)^T [K x M] * G[M x F], without matrix tiles: a 32 x 32 tile would be seven eighths
 * padding along F and the matrix pipes would spend the kernel's time on zeros (114 us for K = 576, F = 3 over 262,144
 * rows). A wavefront owns one source channel and a lane VEC consecutive rows m (samples of one output position): per
 * row vector it loads the F gradient vectors once and the channel's value at each of the TAPS receptor positions, and
 * adds their products into TAPS x F sums of its own; the sums of a slice of M are then added over the 64 lanes (a
 * butterfly of lane exchanges, so every run adds in the same order) and written as the slice's partial [k + K f], k = tap +
 * taps * channel, like the partials of wgrad_body, for the same launch to add. The column sums of G (the bias gradient)
 * come from the first wavefront of every slice. grid = (channels / 4 rounded up, slices).
 * ---------------------------------------------------------------------------------------------- */
template<typename T, int VEC, int MAXT, int NC>
__global__ __launch_bounds__(256)
void few_filters_wgrad_kernel(const T* __restrict__ src, const T* __restrict__ og, T* __restrict__ partials,
		T* __restrict__ bias_partials, const GatherGeom g, int splits, int direct) {
	constexpr int ROWS = 64 * VEC;            /* (NC: accumulators per receptor position, three for an image's, else four) */
	const int lane = threadIdx.x % 64;
	const int wave = __builtin_amdgcn_readfirstlane((int) threadIdx.x / 64);
	const int ch = (int) blockIdx.x * 4 + wave, split = (int) blockIdx.y;
	const int taps = g.R * g.S;
	const bool sums_bias = blockIdx.x == 0 && wave == 0 && bias_partials != nullptr;
	if (ch >= g.LC)
		return;                                  /* (no barrier below) */
	const int total = (g.M + ROWS - 1) / ROWS, per = (total + splits - 1) / splits;
	const int it0 = split * per, it1 = min(total, it0 + per);
	/* the displacement of receptor position t along both axes (wave-uniform, kept in scalar registers) */
	int dya[MAXT], dyb[MAXT];
	#pragma unroll
	for (int t = 0; t < MAXT; ++t) {
		const int tt = min(t, taps - 1);
		dya[t] = (tt % g.R) * g.RA;
		dyb[t] = (tt / g.R) * g.RB;
	}
	T acc[MAXT][NC], bacc[NC];
	#pragma unroll
	for (int t = 0; t < MAXT; ++t)
		#pragma unroll
		for (int f = 0; f < NC; ++f)
			acc[t][f] = (T) 0;
	#pragma unroll
	for (int f = 0; f < NC; ++f)
		bacc[f] = (T) 0;
	const T* const zeros = reinterpret_cast<const T*>(g_zero_block);
	const T* const plane = src + (size_t) g.NS * g.LH * g.LW * ch;
	for (int it = it0; it < it1; ++it) {
		const int m = it * ROWS + lane * VEC;
		const bool valid = m < g.M;              /* whole vectors: M is a multiple of VEC */
		const int n = m % g.N, pos = m / g.N;
		const int a = pos % g.OA, b = pos / g.OA;
		const int ya0 = a * g.SA + g.PA, yb0 = b * g.SB + g.PB;
		T gv[NC][VEC], xv[MAXT][VEC];
		#pragma unroll
		for (int f = 0; f < NC; ++f)
			vec_load_global<T, VEC>(gv[f], valid && f < g.F ? og + ((size_t) m + (size_t) g.M * f) : zeros);
		#pragma unroll
		for (int t = 0; t < MAXT; ++t) {
			const int ya = ya0 + dya[t], yb = yb0 + dyb[t];
			const bool ok = valid && t < taps && (unsigned) ya < (unsigned) g.LH && (unsigned) yb < (unsigned) g.LW;
			vec_load_global<T, VEC>(xv[t], ok ? plane + (n + g.NS * (ya + g.LH * yb)) : zeros);
		}
		#pragma unroll
		for (int t = 0; t < MAXT; ++t)
			#pragma unroll
			for (int f = 0; f < NC; ++f)
				#pragma unroll
				for (int i = 0; i < VEC; ++i)
					acc[t][f] += xv[t][i] * gv[f][i];
		if (sums_bias) {
			#pragma unroll
			for (int f = 0; f < NC; ++f)
				#pragma unroll
				for (int i = 0; i < VEC; ++i)
					bacc[f] += gv[f][i];
		}
	}
	/* the lanes' sums: a butterfly, after which every lane holds the total */
	#pragma unroll
	for (int off = 32; off >= 1; off >>= 1) {
		#pragma unroll
		for (int t = 0; t < MAXT; ++t)
			#pragma unroll
			for (int f = 0; f < NC; ++f)
				acc[t][f] += __shfl_xor(acc[t][f], off, 64);
		#pragma unroll
		for (int f = 0; f < NC; ++f)
			bacc[f] += __shfl_xor(bacc[f], off, 64);
	}
	/* lane t * NC + f writes sum (t, f) */
	T* dst = partials + (size_t) split * ((size_t) g.K * g.F);
	#pragma unroll
	for (int t = 0; t < MAXT; ++t)
		#pragma unroll
		for (int f = 0; f < NC; ++f)
			if (lane == (t * NC + f) % 64 && t < taps && f < g.F) {
				T* o = dst + ((size_t) (t + taps * ch) + (size_t) g.K * f);
				*o = direct ? *o + acc[t][f] : acc[t][f];
			}
	if (sums_bias) {
		#pragma unroll
		for (int f = 0; f < NC; ++f)
			if (lane == f && f < g.F) {
				T* o = bias_partials + ((size_t) split * g.F + f);
				*o = direct ? *o + bacc[f] : bacc[f];
			}
	}
}

/* ------------------------------------------------------------------------------------------------
 * The same product for problems with far fewer output tiles than the chip has wavefront slots, as one launch without
 * partial sums in memory: a block owns one TL x TL tile of the result (one matrix-instruction tile) and its WAVES
 * wavefronts each take a contiguous share of the reduction; their partial tiles meet in LDS and are added in ascending
 * wavefront order, then bias, activation (or the LSTM backward step that consumes the sums) and the store, one output
 * element per thread. Operands go from global memory straight into the operand registers of the matrix instruction (a
 * lane loads the one element per operand that the instruction wants from it: TL consecutive m, or TL consecutive
 * columns of a prepared weight row, per reduction slot - whole 128-byte lines).
 * The reduction runs tap by tap (receptor position), channels innermost, the KS reduction slots of an instruction being
 * KS consecutive channels of one tap: a sum may be taken in any order, and in this one a lane's padding test and
 * position are fixed for a whole tap and a step costs two offset additions, two selects, two loads and the matrix
 * instruction - a wavefront issues one vector instruction per four cycles, and the address arithmetic of a gather by
 * reduction index would outweigh the matrix instruction it feeds. Needs LC % KS == 0.
 * grid = (M tiles rounded up to 8, F tiles).
 * ---------------------------------------------------------------------------------------------- */
enum { WS_PLAIN = 0, WS_ACT = 1, WS_LSTM_BACKWARD = 2 };

template<typename T, int WAVES, bool DIVS, int TAIL>
__global__ __launch_bounds__(64 * WAVES)
void wave_split_gemm_kernel(const T* __restrict__ src, const T* __restrict__ wt, const T* __restrict__ bias, T* __restrict__ out,
		const GatherGeom g, int mtiles, const Epilogue<T> E, const LstmBackwardStep<T> then) {
	typedef Mfma<T> MF;
	constexpr int THREADS = 64 * WAVES;
	constexpr int TL = MF::TL, KS = MF::KS;
	/* Reduction steps per batch of loads: 64 operand registers in fp32, 48 in fp64 (a block of sixteen wavefronts has 128
	 * registers per lane; more spilled), 32 in the blocks of four wavefronts, of which a CU must hold four (measured: at
	 * 136 registers it held three, and 1024 tiles took a second round) */
	/* (the LSTM tail keeps nine preloaded values per lane through the loop: shorter batches make room for them) */
	constexpr int B = sizeof(T) == 4 ? (WAVES == 4 ? 16 : (TAIL == WS_LSTM_BACKWARD ? 24 : 32)) : (WAVES == 4 ? 8 : 12);
	__shared__ T red[WAVES * TL * TL];

	const int mtile = xcd_tile(blockIdx.x, mtiles);
	if (mtile >= mtiles)
		return;
	const int tid = threadIdx.x;
	const int lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
	const int lc = lane % TL, lk = lane / TL;
	const int m0 = mtile * TL, f0 = (int) blockIdx.y * TL;
	const int plane = g.NS * g.LH * g.LW;
	const int m = m0 + lc;
	const bool mvalid = m < g.M;
	int n, ya0, yb0;
	{
		n = m % g.N;
		const int t = m / g.N;
		const int a = t % g.OA, b = t / g.OA;
		ya0 = a * g.SA + g.PA;
		yb0 = b * g.SB + g.PB;
	}
	/* this wavefront's steps of the reduction, numbered tap-major: step = tap * spt + channel group */
	const int taps = g.R * g.S, spt = g.LC / KS;
	const int total = taps * spt;
	const int per = (total + WAVES - 1) / WAVES;
	const int s_begin = wave * per, s_end = min(total, s_begin + per);
	const unsigned astep = (unsigned) (plane * KS) * (unsigned) sizeof(T), bstep = (unsigned) (taps * KS * g.ldw) * (unsigned) sizeof(T);   /* bytes */

	/* LSTM tail: what the backward step of this thread's first output element reads is fetched now and used after the
	 * reduction, so that the kernel does not end with a round trip to memory */
	const int o_first = tid;
	const int mo_first = m0 + o_first % TL, f_first = f0 + o_first / TL;
	bool preloaded = false;
	LstmBackwardInputs<T> pre = {};
	if constexpr (TAIL == WS_LSTM_BACKWARD) {
		preloaded = lstm_backward_can_preload(then);
		const bool mine = o_first < TL * TL && mo_first < g.M && f_first < g.F;
		pre = lstm_backward_load<T>(then, preloaded && mine ? (unsigned) mo_first + (unsigned) g.M * (unsigned) f_first : 0u, true);
	}
	/* one accumulator: a SIMD's matrix pipe runs one instruction at a time, so a chain of dependent instructions costs
	 * nothing, and a second accumulator's registers are worth more as loads in flight */
	typename MF::acc_t acc;
	#pragma unroll
	for (int r = 0; r < MF::NACC; ++r)
		acc[r] = (T) 0;

	for (int s0 = s_begin; s0 < s_end;) {
		const int tap = s0 / spt, cg0 = s0 - tap * spt;
		const int count = min(spt - cg0, s_end - s0);        /* this wavefront's steps inside the tap */
		const int r = tap % g.R, sb = tap / g.R;
		int ya = ya0 + r * g.RA, yb = yb0 + sb * g.RB;
		bool ok = mvalid;
		if (DIVS) {
			const int qa = ya / g.DA, qb = yb / g.DB;
			ok = ok && qa * g.DA == ya && qb * g.DB == yb;
			ya = qa;
			yb = qb;
		}
		ok = ok && (unsigned) ya < (unsigned) g.LH && (unsigned) yb < (unsigned) g.LW;
		const int c_first = cg0 * KS + lk;
		/* 32-bit byte offsets from the kernel's own pointers: a load then needs one address register, not two, and
		 * a whole batch of loads fits beside the accumulators. Lanes in the padding read element 0 and drop it. */
		unsigned aoff = ok ? (unsigned) (n + g.NS * (ya + g.LH * yb) + plane * c_first) * (unsigned) sizeof(T) : 0u;
		const unsigned ainc = ok ? astep : 0u;
		unsigned boff = (unsigned) ((tap + taps * c_first) * g.ldw + f0 + lc) * (unsigned) sizeof(T);
		auto load_a = [&](unsigned off) {
			return *(const __attribute__((address_space(1))) T*) (reinterpret_cast<const char*>(src) + (size_t) off);
		};
		auto load_b = [&](unsigned off) {
			return *(const __attribute__((address_space(1))) T*) (reinterpret_cast<const char*>(wt) + (size_t) off);
		};
		/* Batches of B steps: all of a batch's loads are issued, then its matrix instructions run as the values arrive;
		 * the other wavefronts of the SIMD cover the wait. (Loads of the next batch issued ahead of this one's matrix
		 * instructions were tried: the values carried around the loop cost register copies that wait for every load.) */
		int i = 0;
		for (; i + B <= count; i += B) {
			T xa[B], wb[B];
			#pragma unroll
			for (int u = 0; u < B; ++u) {
				xa[u] = load_a(aoff + (unsigned) u * ainc);
				wb[u] = load_b(boff + (unsigned) u * bstep);
			}
			aoff += B * ainc;
			boff += B * bstep;
			__builtin_amdgcn_sched_barrier(0);
			#pragma unroll
			for (int u = 0; u < B; ++u)
				acc = MF::mma(wb[u], ok ? xa[u] : (T) 0, acc);
			__builtin_amdgcn_sched_barrier(0);
		}
		if (i < count) {
			/* the last, short batch: steps past the end read the last step's addresses again and drop the gathered value */
			const int rem = count - i;
			T xa[B], wb[B];
			#pragma unroll
			for (int u = 0; u < B; ++u) {
				const unsigned uu = (unsigned) min(u, rem - 1);
				xa[u] = load_a(aoff + uu * ainc);
				wb[u] = load_b(boff + uu * bstep);
			}
			__builtin_amdgcn_sched_barrier(0);
			/* (in groups of four, so that a short remainder does not pay for a whole batch of matrix instructions) */
			#pragma unroll
			for (int u0 = 0; u0 < B; u0 += 4)
				if (u0 < rem) {
					#pragma unroll
					for (int u = u0; u < u0 + 4; ++u)
						acc = MF::mma(wb[u], (ok && u < rem) ? xa[u] : (T) 0, acc);
				}
			__builtin_amdgcn_sched_barrier(0);
		}
		s0 += count;
	}
	#pragma unroll
	for (int r = 0; r < MF::NACC; ++r)
		red[(wave * TL + acc_row<T>(r, lk)) * TL + lc] = acc[r];
	__syncthreads();
	for (int o = tid; o < TL * TL; o += THREADS) {
		T v = red[o];
		#pragma unroll
		for (int w = 1; w < WAVES; ++w)
			v += red[w * TL * TL + o];
		const int mo = m0 + o % TL, f = f0 + o / TL;
		if (mo >= g.M || f >= g.F)
			continue;
		if constexpr (TAIL == WS_LSTM_BACKWARD) {
			const unsigned e = (unsigned) mo + (unsigned) g.M * (unsigned) f;
			if (preloaded && o == o_first) {
				if (lstm_standard_acts(then.a))
					lstm_backward_finish<T, true>(then, e, true, v, pre);
				else
					lstm_backward_finish<T, false>(then, e, true, v, pre);
			} else if (lstm_standard_acts(then.a))
				lstm_backward_element<T, true>(then, e, true, v);
			else
				lstm_backward_element<T, false>(then, e, true, v);
		} else {
			v += bias ? bias[f] : (T) 0;
			if constexpr (TAIL == WS_ACT) {
				const size_t at = (size_t) mo + (size_t) g.M * f;
				if (E.pre)
					E.pre[at] = v;
				act_dispatch(E.kind, [&](auto kc) {
					v = act_f_coded<T, decltype(kc)::value>(v, E.p);
				});
				out[at] = v;
			} else {
				out[out_row(g, mo) + (size_t) g.out_M * f] = v;
			}
		}
	}
}

/* out tile = bias + sum over the parts of a split reduction, parts taken in ascending order (so the result
 * does not depend on how blocks were scheduled). One block per (walk position, f block) tile. */
template<typename T, bool ACT>
__global__ __launch_bounds__(256)
void split_reduce_kernel(const T* __restrict__ partials, const T* __restrict__ bias, T* __restrict__ out, const GatherGeom g,
		const GatherLaunch L, int BM, int BF, int ftiles, const Epilogue<T> E) {
	const int M = g.M, F = g.F;
	constexpr int V = 16 / (int) sizeof(T);             /* consecutive m per thread: one 16-byte load per part */
	const int groups = BM * BF / (256 * V);             /* blocks per tile; tiles are multiples of 64 x 32 */
	const int t = blockIdx.x / groups, grp = blockIdx.x % groups;
	const int local = t / ftiles, fb = t % ftiles;
	int tile = L.main_count + local;
	if (L.tile_rows > 0)
		tile = swizzle_tile(tile, L.tile_rows, L.mtiles / L.tile_rows);
	const size_t tile_elems = (size_t) BM * BF;
	const int e = (grp * 256 + threadIdx.x) * V;
	const T* base = partials + (size_t) t * L.ksplit * tile_elems + e;
	T acc[V];
	vec_load<T, V>(acc, base);
	/* eight parts' loads are issued before the first of their additions (a thread's loads are otherwise a chain of
	 * memory round trips, one per part); past the last part the load repeats it and the addition is skipped */
	constexpr int AHEAD = 8;
	for (int z0 = 1; z0 < L.ksplit; z0 += AHEAD) {
		T part[AHEAD][V];
		#pragma unroll
		for (int j = 0; j < AHEAD; ++j)
			vec_load<T, V>(part[j], base + (size_t) min(z0 + j, L.ksplit - 1) * tile_elems);
		#pragma unroll
		for (int j = 0; j < AHEAD; ++j)
			if (z0 + j < L.ksplit) {
				#pragma unroll
				for (int i = 0; i < V; ++i)
					acc[i] += part[j][i];
			}
	}
	const int m = tile_row_m(L, g, tile, BM, e % BM), f = fb * BF + e / BM;
	if (f >= F)
		return;
	const T bv = bias ? bias[f] : (T) 0;
	#pragma unroll
	for (int i = 0; i < V; ++i)
		acc[i] += bv;
	T pre[V];
	if constexpr (ACT) {
		/* the activation epilogue of the whole tiles, applied to the summed parts (EPI_ACT) */
		#pragma unroll
		for (int i = 0; i < V; ++i)
			pre[i] = acc[i];
		act_dispatch(E.kind, [&](auto kc) {
			#pragma unroll
			for (int i = 0; i < V; ++i)
				acc[i] = act_f_coded<T, decltype(kc)::value>(acc[i], E.p);
		});
	}
	const size_t o = ACT ? (size_t) m + (size_t) M * f : out_row(g, min(m, M - 1)) + (size_t) g.out_M * f;
	T* dst = out + o;
	if (m + V <= M && (reinterpret_cast<uintptr_t>(dst) & 15) == 0 && (!ACT || !E.pre || (reinterpret_cast<uintptr_t>(E.pre + o) & 15) == 0)) {
		vec_store_stream<T, V>(dst, acc);
		if constexpr (ACT)
			if (E.pre)
				vec_store_stream<T, V>(E.pre + o, pre);
	} else {
		#pragma unroll
		for (int i = 0; i < V; ++i)
			if (m + i < M) {
				dst[i] = acc[i];
				if constexpr (ACT)
					if (E.pre)
						E.pre[o + i] = pre[i];
			}
	}
}

/* The same sums, taken as the gradient of an LSTM cell's hidden output (the input gradient of the output-side kernels
 * of the step after) and handed, one element per thread, to the element-wise part of the step's backward pass: the
 * gradient tensor itself is never written. */
template<typename T>
__global__ __launch_bounds__(256)
void split_reduce_lstm_backward_kernel(const T* __restrict__ partials, const GatherGeom g, const GatherLaunch L, int BM, int BF,
		int ftiles, const LstmBackwardStep<T> A) {
	const int groups = BM * BF / 256;
	const int t = blockIdx.x / groups, grp = blockIdx.x % groups;
	const int local = t / ftiles, fb = t % ftiles;
	int tile = L.main_count + local;
	if (L.tile_rows > 0)
		tile = swizzle_tile(tile, L.tile_rows, L.mtiles / L.tile_rows);
	const size_t tile_elems = (size_t) BM * BF;
	const int e = grp * 256 + threadIdx.x;
	const T* base = partials + (size_t) t * L.ksplit * tile_elems + e;
	T acc = base[0];
	constexpr int AHEAD = 8;
	for (int z0 = 1; z0 < L.ksplit; z0 += AHEAD) {
		T part[AHEAD];
		#pragma unroll
		for (int j = 0; j < AHEAD; ++j)
			part[j] = base[(size_t) min(z0 + j, L.ksplit - 1) * tile_elems];
		#pragma unroll
		for (int j = 0; j < AHEAD; ++j)
			if (z0 + j < L.ksplit)
				acc += part[j];
	}
	const int m = tile_row_m(L, g, tile, BM, e % BM), f = fb * BF + e / BM;
	if (m >= g.M || f >= g.F)
		return;
	if (lstm_standard_acts(A.a))
		lstm_backward_element<T, true>(A, (unsigned) m + (unsigned) g.M * (unsigned) f, true, acc);
	else
		lstm_backward_element<T, false>(A, (unsigned) m + (unsigned) g.M * (unsigned) f, true, acc);
}

/* A weight-gradient launch of one-wavefront 32 x 32 tiles (fp32) that may ride in an input-gradient launch
 * (gather_with_wgrad_kernel) instead of being a launch of its own; `done` says whether it did. */
template<typename T>
struct WgradRider {
	const T *x, *og;
	T *partials, *bias_partials;
	GatherGeom g;
	WgradSplit plan;
	bool done;
};

/* One instantiation of gather_gemm_kernel and what the tile chooser needs to know about it. */
template<typename T>
struct GatherVariant {
	int bm, bf, waves, lds_bytes;
	int kc;
	void (*launch)(dim3 grid, size_t dyn_lds, const T*, const T*, const T*, T*, const GatherGeom&, const GatherLaunch&,
			T* partials, bool vec, bool divs, int epi, const Epilogue<T>&);
	void (*launch_classes)(dim3 grid, const T* src, T* out, const GatherClasses<T>&);      /* 16-byte loads, no divisors, no epilogue */
	/* whole tiles, 16-byte loads, no divisors, no bias, no epilogue, with a small weight gradient in the same launch; null
	 * where that kernel does not exist */
	void (*launch_with_wgrad)(const GatherLaunch&, int ftiles, const T* src, const T* wt, T* out, const GatherGeom&, const WgradRider<T>&);
	int (*blocks_per_cu)(size_t dyn_lds, bool vec, bool divs, int epi);       /* what the runtime says fits on a CU */
};

/* The fused epilogues exist for the vectorised, divisor-free (forward) form of every tile shape. */
template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int PF>
void launch_gather_variant(dim3 grid, size_t dyn, const T* src, const T* wt, const T* bias, T* out, const GatherGeom& g,
		const GatherLaunch& L, T* partials, bool vec, bool divs, int epi, const Epilogue<T>& E) {
	constexpr int VEC = GemmCfg<T>::VEC;
	dim3 block(64 * WAVES_M * WAVES_F);
	if (epi != EPI_NONE) {
		CATTLE_HIP_REQUIRE(vec && !divs, "a fused epilogue needs the vectorised forward form of the GEMM");
		if (epi == EPI_LSTM) {
			if constexpr (WAVES_M * WT_M <= 128)
				gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_LSTM, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
			else
				throw Error(ERR_INVALID, "the LSTM epilogue exists for the short tiles only");
		} else if (epi == EPI_ACT)
			gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_ACT, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
		else if (epi == EPI_POOL)
			gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_POOL, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
		else
			gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_STATS, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
	} else if (vec && !divs)
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_NONE, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
	else if (vec && divs)
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, true, EPI_NONE, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
	else if (!divs)
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, 1, false, EPI_NONE, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
	else
		gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, 1, true, EPI_NONE, PF><<<grid, block, dyn, stream()>>>(src, wt, bias, out, g, L, partials, E);
	CATTLE_HIP_CHECK(hipGetLastError());
}

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC>
void launch_gather_with_wgrad_variant(const GatherLaunch& L, int ftiles, const T* src, const T* wt, T* out, const GatherGeom& g,
		const WgradRider<T>& r) {
	const int gather_x = L.main_blocks;
	const int w_blocks = round_up(r.plan.tiles * r.plan.splits, 8);
	const dim3 grid((unsigned) (gather_x + (w_blocks + ftiles - 1) / ftiles), (unsigned) ftiles), block(64 * WAVES_M * WAVES_F);
	gather_with_wgrad_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, GemmCfg<T>::VEC><<<grid, block, 0, stream()>>>(src, wt, out, g, L, gather_x,
			r.x, r.og, r.partials, r.bias_partials, r.g, r.plan);
	CATTLE_HIP_CHECK(hipGetLastError());
}

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC>
void launch_gather_classes_variant(dim3 grid, const T* src, T* out, const GatherClasses<T>& classes) {
	gather_gemm_classes_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, GemmCfg<T>::VEC><<<grid, dim3(64 * WAVES_M * WAVES_F), 0, stream()>>>(src, out, classes);
	CATTLE_HIP_CHECK(hipGetLastError());
}

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC, int PF>
int gather_variant_occupancy(size_t dyn, bool vec, bool divs, int epi) {
	constexpr int VEC = GemmCfg<T>::VEC;
	/* the answer for the usual launch (no reserved dynamic LDS) is kept: one query per kernel instantiation */
	static int cached[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
	int& slot = cached[epi != EPI_NONE ? 3 + epi : (vec ? 2 : 0) + (divs ? 1 : 0)];
	if (dyn == 0 && slot > 0)
		return slot;
	int n = 0;
	hipError_t e;
	constexpr int TH = 64 * WAVES_M * WAVES_F;
	if (epi == EPI_LSTM) {
		if constexpr (WAVES_M * WT_M <= 128)
			e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_LSTM, PF>, TH, dyn);
		else
			return 0;
	} else if (epi == EPI_ACT)
		e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_ACT, PF>, TH, dyn);
	else if (epi == EPI_POOL)
		e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_POOL, PF>, TH, dyn);
	else if (epi == EPI_STATS)
		e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_STATS, PF>, TH, dyn);
	else if (vec && !divs)
		e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, false, EPI_NONE, PF>, TH, dyn);
	else if (vec && divs)
		e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, VEC, true, EPI_NONE, PF>, TH, dyn);
	else if (!divs)
		e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, 1, false, EPI_NONE, PF>, TH, dyn);
	else
		e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gather_gemm_kernel<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, 1, true, EPI_NONE, PF>, TH, dyn);
	CATTLE_HIP_CHECK(e);
	if (dyn == 0)
		slot = n;
	return n;
}

template<typename T, int WAVES_M, int WAVES_F, int WT_M, int WT_F, int KC = GemmCfg<T>::KC, int PF = 1>
GatherVariant<T> gather_variant() {
	typedef GemmCfg<T> C;
	static_assert(WT_ROW_PAD % KC == 0 && WAVES_F * WT_F <= WT_COL_PAD, "prepared weights are padded to whole tiles");
	GatherVariant<T> v;
	v.bm = WAVES_M * WT_M;
	v.bf = WAVES_F * WT_F;
	v.waves = WAVES_M * WAVES_F;
	v.lds_bytes = 2 * KC * (v.bm + v.bf + 2 * C::pad(v.bm)) * (int) sizeof(T) + (PF + 2) * KC * 16;
	v.kc = KC;
	v.launch = &launch_gather_variant<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, PF>;
	v.launch_classes = &launch_gather_classes_variant<T, WAVES_M, WAVES_F, WT_M, WT_F, KC>;
	v.launch_with_wgrad = nullptr;
	if constexpr (std::is_same<T, float>::value && WAVES_M * WT_M <= 64 && PF == 1)      /* the short tiles, fp32 */
		v.launch_with_wgrad = &launch_gather_with_wgrad_variant<T, WAVES_M, WAVES_F, WT_M, WT_F, KC>;
	v.blocks_per_cu = &gather_variant_occupancy<T, WAVES_M, WAVES_F, WT_M, WT_F, KC, PF>;
	return v;
}

template<typename T> struct GatherVariants;
template<> struct GatherVariants<float> {
	static constexpr int COUNT = 9, LARGE = 4, SHORT = 2, TALL32 = 8;
	static const GatherVariant<float>* get() {
		static const GatherVariant<float> v[COUNT] = {
			gather_variant<float, 4, 2, 64, 64>(),      /* 256 x 128 */
			gather_variant<float, 4, 2, 64, 32>(),      /* 256 x 64: eight waves of 64 x 32 beat four of 64 x 64 by 5 % */
			gather_variant<float, 4, 1, 64, 32>(),      /* 256 x 32 */
			gather_variant<float, 8, 1, 64, 64>(),      /* 512 x 64 for very tall problems: eight waves of 64 x 64, 1 % over 256 x 64 */
			/* small problems (a few thousand rows): short tiles so that every CU gets a block, and long
			 * reduction chunks because with one block per CU only the loads in flight hide memory latency */
			gather_variant<float, 2, 2, 32, 32, 64>(),  /* 64 x 64 */
			gather_variant<float, 2, 1, 32, 32, 64>(),  /* 64 x 32 */
			gather_variant<float, 2, 2, 32, 32, 32>(),  /* 64 x 64, chunks of 32: several short tiles per CU */
			gather_variant<float, 2, 1, 32, 32, 32>(),  /* 64 x 32, chunks of 32 */
			gather_variant<float, 4, 1, 32, 32, 32>(),  /* 128 x 32, four waves: few columns, a few hundred tiles */
		};
		return v;
	}
};
template<> struct GatherVariants<double> {
	static constexpr int COUNT = 7, LARGE = 3, SHORT = 2, TALL32 = -1;
	static const GatherVariant<double>* get() {
		static const GatherVariant<double> v[COUNT] = {
			gather_variant<double, 8, 2, 32, 64>(),     /* 256 x 128, sixteen waves */
			gather_variant<double, 4, 2, 64, 32>(),     /* 256 x 64 */
			gather_variant<double, 4, 1, 64, 32>(),     /* 256 x 32 */
			gather_variant<double, 2, 2, 32, 32, 32>(), /* 64 x 64, small problems */
			gather_variant<double, 2, 1, 32, 32, 32>(), /* 64 x 32 */
			gather_variant<double, 2, 2, 32, 32, 16>(), /* 64 x 64, chunks of 16: several short tiles per CU */
			gather_variant<double, 2, 1, 32, 32, 16>(), /* 64 x 32, chunks of 16 */
		};
		return v;
	}
};

/* Switches for experiments. A build with -DCATTLE_HIP_EXPERIMENTS reads them from the environment once, when the first
 * GEMM is launched; the library as shipped has none of them and always takes the launch plan its rules give:
 *   CATTLE_HIP_GATHER_VARIANT_F<F> = index into the gather variant table for GEMMs with F output columns,
 *   CATTLE_HIP_GATHER_OCC_F<F>     = blocks per CU for them (enforced by reserving dynamic LDS),
 *   CATTLE_HIP_NO_SWIZZLE, CATTLE_HIP_NO_ROW_BLOCKS, CATTLE_HIP_NO_SPLIT: tile walk, blocked tile rows, cut reductions off,
 *   CATTLE_HIP_WGRAD_VARIANT, CATTLE_HIP_WGRAD_SPLITS, CATTLE_HIP_WGRAD_LINEAR, CATTLE_HIP_WGRAD_MIN_CHUNKS: the weight-gradient plan. */
struct Tuning {
	struct PerF { int F, variant, occ; };
	std::vector<PerF> per_f;
	bool no_swizzle = false, no_row_blocks = false, no_split = false, wgrad_linear = false, no_wave_split = false;
	int wgrad_variant = -1, wgrad_splits = 0, wgrad_min_chunks = 0;

	Tuning() {
#ifdef CATTLE_HIP_EXPERIMENTS
		no_swizzle = std::getenv("CATTLE_HIP_NO_SWIZZLE") != nullptr;
		no_row_blocks = std::getenv("CATTLE_HIP_NO_ROW_BLOCKS") != nullptr;
		no_split = std::getenv("CATTLE_HIP_NO_SPLIT") != nullptr;
		no_wave_split = std::getenv("CATTLE_HIP_NO_WAVE_SPLIT") != nullptr;
		wgrad_linear = std::getenv("CATTLE_HIP_WGRAD_LINEAR") != nullptr;
		const char* e = std::getenv("CATTLE_HIP_WGRAD_VARIANT");
		wgrad_variant = e ? std::atoi(e) : -1;
		e = std::getenv("CATTLE_HIP_WGRAD_SPLITS");
		wgrad_splits = e ? std::atoi(e) : 0;
		e = std::getenv("CATTLE_HIP_WGRAD_MIN_CHUNKS");
		wgrad_min_chunks = e ? std::atoi(e) : 0;
		for (char** v = environ; v && *v; ++v) {
			static const char* const keys[2] = { "CATTLE_HIP_GATHER_VARIANT_F", "CATTLE_HIP_GATHER_OCC_F" };
			for (int k = 0; k < 2; ++k) {
				const size_t len = std::strlen(keys[k]);
				if (std::strncmp(*v, keys[k], len) != 0)
					continue;
				const char* eq = std::strchr(*v + len, '=');
				if (!eq)
					continue;
				PerF& slot = entry(std::atoi(*v + len));
				(k == 0 ? slot.variant : slot.occ) = std::atoi(eq + 1);
			}
		}
#endif
	}
	PerF& entry(int F) {
		for (PerF& p : per_f)
			if (p.F == F)
				return p;
		per_f.push_back(PerF{ F, -1, 0 });
		return per_f.back();
	}
	const PerF* find(int F) const {
		for (const PerF& p : per_f)
			if (p.F == F)
				return &p;
		return nullptr;
	}
};

const Tuning& tuning() {
	static const Tuning t;
	return t;
}

/* Picks the tile shape: the narrowest F tile that covers all output columns in one block column (so
 * the gathered A operand, the expensive one, is read once), else the widest. Blocks run at the
 * occupancy their LDS and register use allows; measured on MI355X, more co-resident blocks beat
 * fewer blocks even when the last round of blocks is mostly idle. */
/* The blocked tile order (tile_row_m) for tiles of bm rows: SB = 2^sb_shift samples x a pa x pos_b rectangle of
 * output positions. With a pooling epilogue (prh x prw windows, stride = receptor) the rectangle must hold whole
 * windows, and SB may shrink below 32 so that a tile holds at least one. */
struct RowBlocks {
	bool ok;
	int sb_shift, sample_blocks, pos_b, tile_rows;
};

template<typename T>
RowBlocks plan_row_blocks(const GatherGeom& g, int bm, int prh, int prw, bool pooled) {
	RowBlocks rb = { false, 5, 0, 1, 0 };
	const int min_shift = GemmCfg<T>::VEC == 4 ? 2 : 1;           /* a 16-byte access stays inside one sample block */
	for (int shift = 5; shift >= (pooled ? min_shift : 5); --shift) {
		const int sb = 1 << shift;
		if (g.N % sb != 0 || bm % sb != 0)
			continue;
		const int positions = bm / sb;
		for (int pb = prw; pb <= positions; pb *= 2) {
			const int pa = positions / pb;
			if (positions % pb == 0 && pa % prh == 0 && g.OA % pa == 0 && g.OB % pb == 0 && (pooled || g.OB / pb > 1)) {
				rb.ok = true;
				rb.sb_shift = shift;
				rb.sample_blocks = g.N / sb;
				rb.pos_b = pb;
				rb.tile_rows = rb.sample_blocks * (g.OA / pa);
				return rb;
			}
		}
	}
	return rb;
}

/* Picks the tile shape: the narrowest F tile that covers all output columns in one block column (so
 * the gathered A operand, the expensive one, is read once), else the widest. Blocks run at the
 * occupancy their LDS and register use allows; measured on MI355X, more co-resident blocks beat
 * fewer blocks even when the last round of blocks is mostly idle.
 * With a fused epilogue (epi != EPI_NONE; `E` its arguments) the launch needs 16-byte accesses; the pooling and the
 * moments epilogue need whole tiles in one block (no cut reductions), the pooling epilogue the blocked tile order
 * with whole windows per tile. Returns false, without launching, when the problem does not allow that; `mtiles_out`
 * receives the number of M tiles (the row count of the moments epilogue's partials). */
/* Whether, and with how many wavefronts per block, a problem runs as wave_split_gemm_kernel: few enough tiles of one
 * matrix instruction that they and their wavefronts fit the chip at once (sixteen wavefronts per CU), a reduction long
 * enough to deal out, and operand traffic (every tile reads its TL rows of both operands whole) that the L2 caches carry in
 * a few microseconds. 0 = no. */
template<typename T>
int wave_split_waves(const GatherGeom& g) {
	constexpr int TL = Mfma<T>::TL, KS = Mfma<T>::KS;
	const long tiles = (long) ((g.M + TL - 1) / TL) * ((g.F + TL - 1) / TL);
	const long slots = (long) device_shape().cus * 16;
	if (g.LC % KS != 0 || g.LC < 4 * KS || tiles * 4 > slots)
		return 0;
	const int steps = g.K / KS;
	if (steps < 32)
		return 0;
	if (((double) g.R * g.S * g.LC + 64) * g.ldw * sizeof(T) >= 4294967296.0 || (double) g.NS * g.LH * g.LW * g.LC * sizeof(T) >= 4294967296.0)
		return 0;               /* 32-bit byte offsets */
	int waves = 16;
	while (waves > 4 && (tiles * waves > slots || steps < 8 * waves))
		waves /= 2;
	/* A wavefront's share of the reduction is a chain of batches of loads, each a round trip to memory of two
	 * microseconds or more: 48 steps (two or three batches) where the wavefronts are few and their round trips coincide, 80
	 * where the chip is full of them (blocks at different points of their chains overlap). Longer reductions are cut across blocks
	 * (measured: a dense layer 4096 -> 10 at batch 128, four tiles, 23 us this way, 12 us cut across blocks). */
	const int per_wave = (steps + waves - 1) / waves;
	if (per_wave > (tiles * waves * 2 <= slots ? 48 : 80))
		return 0;
	return waves;
}

template<typename T, int WAVES>
void launch_wave_split_variant(const T* src, const T* wt, const T* bias, T* out, const GatherGeom& g, bool divs, int tail,
		const Epilogue<T>& E, const LstmBackwardStep<T>* then) {
	constexpr int TL = Mfma<T>::TL;
	const int mtiles = (g.M + TL - 1) / TL, ftiles = (g.F + TL - 1) / TL;
	const dim3 grid((unsigned) round_up(mtiles, 8), (unsigned) ftiles), block(64 * WAVES);
	const size_t lds = 0;
	LstmBackwardStep<T> none;
	std::memset(&none, 0, sizeof none);
	if (tail == WS_LSTM_BACKWARD)
		wave_split_gemm_kernel<T, WAVES, false, WS_LSTM_BACKWARD><<<grid, block, lds, stream()>>>(src, wt, bias, out, g, mtiles, E, *then);
	else if (tail == WS_ACT)
		wave_split_gemm_kernel<T, WAVES, false, WS_ACT><<<grid, block, lds, stream()>>>(src, wt, bias, out, g, mtiles, E, none);
	else if (divs)
		wave_split_gemm_kernel<T, WAVES, true, WS_PLAIN><<<grid, block, lds, stream()>>>(src, wt, bias, out, g, mtiles, E, none);
	else
		wave_split_gemm_kernel<T, WAVES, false, WS_PLAIN><<<grid, block, lds, stream()>>>(src, wt, bias, out, g, mtiles, E, none);
	CATTLE_HIP_CHECK(hipGetLastError());
}

template<typename T>
bool launch_gather(const T* src, const T* wt, const T* bias, T* out, const GatherGeom& g, ScratchArena* arena = nullptr,
		int epi = EPI_NONE, const Epilogue<T>* E = nullptr, int* mtiles_out = nullptr, const LstmBackwardStep<T>* then = nullptr,
		bool* then_done = nullptr, const std::function<void(int bf)>* before_launch = nullptr, WgradRider<T>* rider = nullptr) {
	const bool vec = g.N % GemmCfg<T>::VEC == 0 && g.NS % GemmCfg<T>::VEC == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0;
	const bool divs = g.DA != 1 || g.DB != 1;
	if (epi != EPI_NONE && (!vec || divs || (reinterpret_cast<uintptr_t>(out) & 15) != 0))
		return false;
	/* 16-byte loads wherever alignment allows, even where they leave a SIMD a wave or two: measured, a quarter of
	 * the load instructions beats four times the waves (9 against 19 us on a 200,704 x 48 x 1 problem) */
	const bool wide = vec && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
	if ((epi == EPI_NONE || epi == EPI_ACT) && then == nullptr && (g.F <= FEW_COLUMNS || (g.F <= SOME_COLUMNS && wide && !divs))) {
		/* a handful of output columns: no matrix tiles (few_columns_gather_kernel); five to eight of them in the
		 * vectorised forward form only */
		constexpr int V = GemmCfg<T>::VEC;
		const unsigned blocks = (unsigned) round_up((g.M + (wide ? 64 * V : 64) - 1) / (wide ? 64 * V : 64), 8);   /* few_columns_block */
		/* how a wave walks the reduction (few_columns_body): with up to eight source channels, steps of all taps in batches
		 * (0); else tap by tap with a wave's share of the channels in whole batches of loads, eight to a batch if that
		 * divides the share, else four */
		const int walk = !divs && wide && g.LC <= 8 ? 0 : ((g.LC + 3) / 4) % 8 == 0 ? 8 : 4;
		/* as many accumulators per row as there are columns, for the counts that images have (one, three), else four or
		 * eight: a fourth accumulator for three columns is a third more multiply-adds */
		const auto with_walk = [&](auto fn) {
			if (walk == 0) fn(std::integral_constant<int, 0>());
			else if (walk == 8) fn(std::integral_constant<int, 8>());
			else fn(std::integral_constant<int, 4>());
		};
		const auto with_columns = [&](auto fn) {
			if (g.F > FEW_COLUMNS) fn(std::integral_constant<int, SOME_COLUMNS>());
			else if (g.F == 3) fn(std::integral_constant<int, 3>());
			else if (g.F == 1) fn(std::integral_constant<int, 1>());
			else fn(std::integral_constant<int, FEW_COLUMNS>());
		};
		/* the activation epilogue (it comes with 16-byte accesses and without divisors, see above) */
		const int act_kind = epi == EPI_ACT ? E->kind : -1;
		const T act_p = epi == EPI_ACT ? E->p : (T) 0;
		T* const act_pre = epi == EPI_ACT ? E->pre : nullptr;
		if (epi == EPI_ACT && (reinterpret_cast<uintptr_t>(act_pre) & 15) != 0)
			return false;
		if (epi == EPI_NONE && g.F <= FEW_COLUMNS && rider && wide && !divs && bias == nullptr) {
			const unsigned w_blocks = (unsigned) round_up(rider->plan.tiles * rider->plan.splits, 8);
			with_walk([&](auto w) {
				if (g.F == 3)
					few_columns_with_wgrad_kernel<T, V, decltype(w)::value, 3><<<blocks + w_blocks, 256, 0, stream()>>>(src, wt, out, g, (int) blocks,
							rider->x, rider->og, rider->partials, rider->bias_partials, rider->g, rider->plan);
				else
					few_columns_with_wgrad_kernel<T, V, decltype(w)::value, FEW_COLUMNS><<<blocks + w_blocks, 256, 0, stream()>>>(src, wt, out, g,
							(int) blocks, rider->x, rider->og, rider->partials, rider->bias_partials, rider->g, rider->plan);
			});
			rider->done = true;
		} else if (wide && divs)
			few_columns_gather_kernel<T, V, true, 8><<<blocks, 256, 0, stream()>>>(src, wt, bias, out, g);
		else if (wide)
			with_walk([&](auto w) {
				with_columns([&](auto c) {
					few_columns_plain_kernel<T, V, decltype(w)::value, decltype(c)::value><<<blocks, 256, 0, stream()>>>(src, wt, bias, out, g,
							act_kind, act_p, act_pre);
				});
			});
		else if (divs)
			few_columns_gather_kernel<T, 1, true, 8><<<blocks, 256, 0, stream()>>>(src, wt, bias, out, g);
		else
			few_columns_gather_kernel<T, 1, false, 8><<<blocks, 256, 0, stream()>>>(src, wt, bias, out, g);
		CATTLE_HIP_CHECK(hipGetLastError());
		if (mtiles_out)
			*mtiles_out = 0;
		return true;
	}
	const GatherVariant<T>* vars = GatherVariants<T>::get();
	int best_v = 0;
	for (int i = 1; i < GatherVariants<T>::LARGE; ++i) {
		const bool narrower = vars[i].bf >= g.F && vars[i].bf < vars[best_v].bf;
		/* same width, taller tile: half the A-operand loads per MFMA; worth it once it still fills the chip */
		const bool taller = vars[i].bf == vars[best_v].bf && vars[i].bm > vars[best_v].bm && g.M >= vars[i].bm * device_shape().cus * 4;
		if (narrower || taller)
			best_v = i;
	}
	/* The widest shape with at most one and a half blocks per CU: the next narrower one doubles the blocks, and with
	 * them the blocks that overlap each other's memory waits on a CU (the input-side LSTM gates, 320 tiles of
	 * 256 x 128 with K = 72: 37 -> 31 us). */
	if (best_v == 0 && vars[0].bf > vars[1].bf && g.F > vars[1].bf) {
		const long blocks = (long) ((g.M + vars[0].bm - 1) / vars[0].bm) * ((g.F + vars[0].bf - 1) / vars[0].bf);
		if (blocks >= device_shape().cus && blocks * 2 <= 3 * device_shape().cus)
			best_v = 1;
	}
	/* (the same one step further down: 86,400 x 216 x 48 on 338 tiles of 256 x 64, 46.6 us; on 676 of 256 x 32, 36.4) */
	if (best_v == 1 && vars[2].bm == vars[1].bm && vars[1].bf > vars[2].bf && g.F > vars[2].bf) {
		const long blocks = (long) ((g.M + vars[1].bm - 1) / vars[1].bm) * ((g.F + vars[1].bf - 1) / vars[1].bf);
		if (blocks >= device_shape().cus && blocks * 2 <= 3 * device_shape().cus)
			best_v = 2;
	}
	/* Too few tiles of that shape to give every CU one: a narrower tile of the same height first, if that does and the
	 * reduction is short. Such a launch is one round of blocks whose time is latency, so two half-width blocks on a CU
	 * overlap each other's waits (50,176 x 576 x 128: 109 -> 96 us), while with a long reduction the matrix pipes are
	 * busy either way and the wider tile's better operand reuse wins (12,544 x 4608 x 512: 624 against 675 us). No
	 * narrower than 64 columns: the 256 x 32 tile, one wave per 64 rows, loses to the short tiles (32,768 x 288 x 64:
	 * 32 against 20 us) ... */
	auto tiles_with = [&](int i) {
		return (long) ((g.M + vars[i].bm - 1) / vars[i].bm) * ((g.F + vars[i].bf - 1) / vars[i].bf);
	};
	if (tiles_with(best_v) < device_shape().cus && epi != EPI_LSTM && g.K <= 1024)
		for (int i = best_v + 1; i < GatherVariants<T>::LARGE; ++i)
			if (vars[i].bm == vars[best_v].bm && vars[i].bf < vars[best_v].bf && vars[i].bf >= 64 && tiles_with(i) >= device_shape().cus) {
				best_v = i;
				break;
			}
	/* ... else the short tiles (the narrowest that still covers F, else the widest) */
	if ((long) ((g.M + vars[best_v].bm - 1) / vars[best_v].bm) * ((g.F + vars[best_v].bf - 1) / vars[best_v].bf) < device_shape().cus) {
		constexpr int SHORT = GatherVariants<T>::SHORT;       /* short shapes, each with long and with medium chunks */
		best_v = GatherVariants<T>::LARGE;
		for (int i = GatherVariants<T>::LARGE + 1; i < GatherVariants<T>::LARGE + SHORT; ++i)
			if (vars[i].bf >= g.F && vars[i].bf < vars[best_v].bf)
				best_v = i;
		/* enough short tiles for two or more per CU: the medium chunks, whose smaller LDS footprint lets four
		 * blocks share a CU. Tiles for at most half of the CUs: the medium chunks too, because the reduction of every
		 * tile is then cut into parts and shorter chunks give twice as many parts to fill the chip with. In between:
		 * the long chunks, with which one block keeps more loads in flight */
		const long short_tiles = (long) ((g.M + vars[best_v].bm - 1) / vars[best_v].bm) * ((g.F + vars[best_v].bf - 1) / vars[best_v].bf);
		if (short_tiles >= 2 * device_shape().cus || short_tiles * 2 <= device_shape().cus)
			best_v += SHORT;
		/* 32 columns and enough rows for every CU to get a tile twice as tall: four waves share the table and the
		 * barriers that two-wave blocks pay for alone (config 3's second input gradient, 512 tiles of 64 x 32 with
		 * K = 576: 33 -> 25 us) */
		if (GatherVariants<T>::TALL32 >= 0 && vars[best_v].bf == 32 &&
				(long) ((g.M + 127) / 128) * ((g.F + 31) / 32) >= device_shape().cus)
			best_v = GatherVariants<T>::TALL32;
	}
	const Tuning& tune = tuning();
	int occ = 0;
	if (const Tuning::PerF* o = tune.find(g.F)) {
		if (o->variant >= 0 && o->variant < GatherVariants<T>::COUNT)
			best_v = o->variant;
		occ = o->occ;
	}
	const bool pooled = epi == EPI_POOL;
	RowBlocks rb = { false, 5, 0, 1, 0 };
	if (pooled) {
		/* the chosen shape if whole windows fit its tiles, else the same width with the other height */
		rb = plan_row_blocks<T>(g, vars[best_v].bm, E->prh, E->prw, true);
		for (int i = 0; !rb.ok && i < GatherVariants<T>::COUNT; ++i)
			if (vars[i].bf == vars[best_v].bf && vars[i].bm != vars[best_v].bm && vars[i].bm <= 256) {
				rb = plan_row_blocks<T>(g, vars[i].bm, E->prh, E->prw, true);
				if (rb.ok)
					best_v = i;
			}
		if (!rb.ok)
			return false;
	}
	const GatherVariant<T>& v = vars[best_v];
	if (epi == EPI_LSTM) {
		/* a short tile (it stages itself whole) whose column groups are whole gate groups of the hidden channels */
		const int hidden = g.F / 4;
		if (v.bm > 128 || g.F % 4 != 0 || hidden % (v.bf / 4) != 0 || (size_t) g.M * hidden != E->lstm.P ||
				!lstm_forward_vectors<T>(E->lstm, GemmCfg<T>::VEC))
			return false;
	}
	if (before_launch)
		(*before_launch)(v.bf);
	size_t dyn = 0;
	if (occ >= 1 && occ <= 8) {
		const int want_bytes = device_shape().lds_per_cu / (occ + 1) + 256;
		dyn = want_bytes > v.lds_bytes ? (size_t) (want_bytes - v.lds_bytes) : 0;
	}
	const int mtiles = (g.M + v.bm - 1) / v.bm, ftiles = (g.F + v.bf - 1) / v.bf;
	const int nchunks = (g.K + v.kc - 1) / v.kc;
	/* tiles per output column, if a column (N * OA rows of M) is a whole number of tiles and there are
	 * several columns; 0 switches the 2-D walk off */
	const long column = (long) g.N * g.OA;
	int tile_rows = (column % v.bm == 0 && g.OB > 1 && !tune.no_swizzle && !pooled) ? (int) (column / v.bm) : 0;
	/* rows of a tile as 32 samples x a rectangle of positions (see tile_row_m) where the shape allows it: as many
	 * positions along a as divide OA, the rest along b; the 2-D walk then runs over strips of pos_b columns */
	int sample_blocks = 0, pos_b = 1, sb_shift = 5;
	if (pooled) {
		sample_blocks = rb.sample_blocks;
		pos_b = rb.pos_b;
		tile_rows = rb.tile_rows;
		sb_shift = rb.sb_shift;
	} else if (g.N % 32 == 0 && v.bm % 32 == 0 && g.OB > 1 && !tune.no_swizzle && !tune.no_row_blocks) {
		rb = plan_row_blocks<T>(g, v.bm, 1, 1, false);
		if (rb.ok) {
			sample_blocks = rb.sample_blocks;
			pos_b = rb.pos_b;
			tile_rows = rb.tile_rows;
		}
	}
	if (mtiles_out)
		*mtiles_out = mtiles;
	/* blocks the chip holds at once (registers, LDS, waves), as the runtime computes it for this kernel */
	const int per_cu = std::max(1, v.blocks_per_cu(dyn, vec, divs, epi));
	const int slots = device_shape().cus * per_cu;
	const bool no_split = tune.no_split || epi == EPI_POOL || epi == EPI_STATS || epi == EPI_LSTM;
	const Epilogue<T> none = { 0, (T) 0, nullptr, nullptr, 1, 1, 1, 1, nullptr, {} };
	const Epilogue<T>& epi_args = E ? *E : none;

	/* main_count whole tiles, the other mtiles - main_count with their reduction cut into about `ksplit` parts */
	auto launch = [&](int main_count, int ksplit) {
		GatherLaunch L = { mtiles, tile_rows, main_count, round_up(main_count, 8), mtiles - main_count, 1, nchunks, sample_blocks, pos_b, sb_shift };
		T* partials = nullptr;
		if (L.split_count > 0) {
			L.chunks_per_part = (nchunks + ksplit - 1) / ksplit;
			L.ksplit = (nchunks + L.chunks_per_part - 1) / L.chunks_per_part;       /* no empty part */
			const size_t pbytes = (size_t) L.split_count * ftiles * L.ksplit * v.bm * v.bf * sizeof(T);
			partials = static_cast<T*>(arena ? arena->take(pbytes, "partial sums of the split reduction") : split_workspace(pbytes));
		}
		dim3 grid((unsigned) (L.main_blocks + L.split_count * L.ksplit), (unsigned) ftiles);
		v.launch(grid, dyn, src, wt, bias, out, g, L, partials, vec, divs, epi, epi_args);
		if (L.split_count > 0) {
			const int groups = v.bm * v.bf / (256 * (16 / (int) sizeof(T)));
			const dim3 rgrid((unsigned) (L.split_count * ftiles * groups));
			if (then && main_count == 0 && bias == nullptr && epi == EPI_NONE && (size_t) g.M * g.F == then->P) {
				const dim3 egrid((unsigned) (L.split_count * ftiles * (v.bm * v.bf / 256)));
				split_reduce_lstm_backward_kernel<T><<<egrid, 256, 0, stream()>>>(partials, g, L, v.bm, v.bf, ftiles, *then);
				*then_done = true;
			} else if (epi == EPI_ACT)
				split_reduce_kernel<T, true><<<rgrid, 256, 0, stream()>>>(partials, bias, out, g, L, v.bm, v.bf, ftiles, epi_args);
			else
				split_reduce_kernel<T, false><<<rgrid, 256, 0, stream()>>>(partials, bias, out, g, L, v.bm, v.bf, ftiles, epi_args);
			CATTLE_HIP_CHECK(hipGetLastError());
		}
	};

	const long total = (long) mtiles * ftiles;
	if (!no_split && total * 2 <= slots && nchunks >= 4) {
		/* far fewer tiles than the chip holds blocks: the reduction of every tile is dealt to the wavefronts of one block
		 * where it is short enough for that (wave_split_gemm_kernel: one launch, no partial sums in memory), else cut into
		 * parts, one block each, which a second launch adds up */
		const bool lstm_tail = then != nullptr && epi == EPI_NONE && bias == nullptr && (size_t) g.M * g.F == then->P;
		const int tail = lstm_tail ? WS_LSTM_BACKWARD : epi == EPI_ACT ? WS_ACT : WS_PLAIN;
		const int waves = ((divs && tail != WS_PLAIN) || tune.no_wave_split) ? 0 : wave_split_waves<T>(g);
		if (waves > 0) {
			if (waves == 16)
				launch_wave_split_variant<T, 16>(src, wt, bias, out, g, divs, tail, epi_args, then);
			else if (waves == 8)
				launch_wave_split_variant<T, 8>(src, wt, bias, out, g, divs, tail, epi_args, then);
			else
				launch_wave_split_variant<T, 4>(src, wt, bias, out, g, divs, tail, epi_args, then);
			if (lstm_tail)
				*then_done = true;
			return true;
		}
		launch(0, (int) std::min<long>(std::min<long>(slots / total, nchunks / 2), 32));
		return true;
	}
	/* (a round of the chip holds slots / ftiles rows of tiles) */
	const int round_m = std::max(1, slots / ftiles), rem = mtiles % round_m;
	if (!no_split && mtiles > round_m && rem > 0 && rem * 2 <= round_m && nchunks >= 8) {
		/* The tiles left over after whole rounds would keep a fraction of the chip busy for a whole tile time.
		 * Their reduction is cut into parts instead; the part blocks come last in the grid and fill the
		 * chip as the last round of whole tiles drains. */
		launch(mtiles - rem, (int) std::min<long>(std::min(round_m / rem, nchunks / 4), 16));
		return true;
	}
	if (rider && v.launch_with_wgrad && epi == EPI_NONE && bias == nullptr && then == nullptr && vec && !divs && dyn == 0 &&
			g.out_sa == 1 && g.out_sb == 1 && g.out_a0 == 0 && g.out_b0 == 0 && g.out_OA == g.OA && g.out_M == g.M) {
		/* whole tiles only, and a small weight gradient that waits for the same upstream gradient: one launch for both */
		const GatherLaunch L = { mtiles, tile_rows, mtiles, round_up(mtiles, 8), 0, 1, nchunks, sample_blocks, pos_b, sb_shift };
		v.launch_with_wgrad(L, ftiles, src, wt, out, g, *rider);
		rider->done = true;
		return true;
	}
	launch(mtiles, 1);
	return true;
}

/* All problems of `geoms` (same source, same result tensor, same column count; 16-byte loads possible) as one launch
 * whose third grid dimension is the problem. The tile shape is chosen for the tiles of all problems together - a class
 * of a strided input gradient alone may have too few rows for the large tiles that the whole gradient fills the chip
 * with. Returns false, having launched nothing, if there are more problems than the table holds. */
template<typename T>
bool launch_gather_classes(const T* src, T* out, const std::vector<GatherGeom>& geoms, const std::vector<const T*>& weights) {
	if (geoms.empty())
		return true;
	if ((int) geoms.size() > MAX_GATHER_CLASSES)
		return false;
	const GatherVariant<T>* vars = GatherVariants<T>::get();
	const int F = geoms[0].F;
	auto tiles_of = [&](const GatherVariant<T>& v) {
		long t = 0;
		for (const GatherGeom& g : geoms)
			t += (long) ((g.M + v.bm - 1) / v.bm) * ((F + v.bf - 1) / v.bf);
		return t;
	};
	/* the narrowest large tile that covers all columns in one block column, else the widest; the short tiles if the
	 * large ones would not give every CU a block */
	int best_v = 0;
	for (int i = 1; i < GatherVariants<T>::LARGE; ++i)
		if (vars[i].bm == vars[0].bm && vars[i].bf >= F && vars[i].bf < vars[best_v].bf)
			best_v = i;
	if (tiles_of(vars[best_v]) < device_shape().cus)
		for (int i = best_v + 1; i < GatherVariants<T>::LARGE; ++i)
			if (vars[i].bm == vars[best_v].bm && vars[i].bf < vars[best_v].bf && vars[i].bf >= 64 && tiles_of(vars[i]) >= device_shape().cus) {
				best_v = i;
				break;
			}
	if (tiles_of(vars[best_v]) < device_shape().cus) {
		constexpr int SHORT = GatherVariants<T>::SHORT;
		best_v = GatherVariants<T>::LARGE;
		for (int i = GatherVariants<T>::LARGE + 1; i < GatherVariants<T>::LARGE + SHORT; ++i)
			if (vars[i].bf >= F && vars[i].bf < vars[best_v].bf)
				best_v = i;
		if (tiles_of(vars[best_v]) >= 2 * device_shape().cus)
			best_v += SHORT;                /* several short tiles per CU: the medium chunks, four blocks to a CU */
	}
	const GatherVariant<T>& v = vars[best_v];
	GatherClasses<T> table;
	unsigned blocks = 0;
	for (size_t i = 0; i < geoms.size(); ++i) {
		const GatherGeom& g = geoms[i];
		const int mtiles = (g.M + v.bm - 1) / v.bm;
		const long column = (long) g.N * g.OA;
		int tile_rows = (column % v.bm == 0 && g.OB > 1) ? (int) (column / v.bm) : 0;
		int sample_blocks = 0, pos_b = 1;
		if (g.N % 32 == 0 && v.bm % 32 == 0 && g.OB > 1) {
			const RowBlocks rb = plan_row_blocks<T>(g, v.bm, 1, 1, false);
			if (rb.ok) {
				sample_blocks = rb.sample_blocks;
				pos_b = rb.pos_b;
				tile_rows = rb.tile_rows;
			}
		}
		table.g[i] = g;
		table.L[i] = GatherLaunch{ mtiles, tile_rows, mtiles, round_up(mtiles, 8), 0, 1, (g.K + v.kc - 1) / v.kc, sample_blocks, pos_b, 5 };
		table.wt[i] = weights[i];
		blocks = std::max(blocks, (unsigned) round_up(mtiles, 8));
	}
	for (size_t i = geoms.size(); i < (size_t) MAX_GATHER_CLASSES; ++i) {
		table.g[i] = geoms[0];
		table.L[i] = table.L[0];
		table.wt[i] = weights[0];
	}
	v.launch_classes(dim3(blocks, (unsigned) ((F + v.bf - 1) / v.bf), (unsigned) geoms.size()), src, out, table);
	return true;
}

void plain_output(GatherGeom& g) {
	g.out_a0 = g.out_b0 = 0;
	g.out_sa = g.out_sb = 1;
	g.out_OA = g.OA;
	g.out_M = g.M;
}

GatherGeom forward_geom(const ConvShape& s, int N) {
	GatherGeom g;
	g.N = N; g.NS = N; g.LH = s.H; g.LW = s.W; g.LC = s.C;
	g.OA = s.OH(); g.OB = s.OW();
	g.R = s.RH; g.S = s.RW;
	g.SA = s.sv; g.SB = s.sh; g.RA = s.dv + 1; g.RB = s.dh + 1; g.PA = -s.pv; g.PB = -s.ph; g.DA = 1; g.DB = 1;
	g.M = N * g.OA * g.OB; g.K = s.K(); g.F = s.F;
	g.ldw = round_up(s.F, WT_COL_PAD);
	plain_output(g);
	return g;
}

GatherGeom dgrad_geom(const ConvShape& s, int N) {
	GatherGeom g;
	g.N = N; g.NS = N; g.LH = s.OH(); g.LW = s.OW(); g.LC = s.F;
	g.OA = s.H; g.OB = s.W;
	g.R = s.RH; g.S = s.RW;
	g.SA = 1; g.SB = 1; g.RA = -(s.dv + 1); g.RB = -(s.dh + 1); g.PA = s.pv; g.PB = s.ph; g.DA = s.sv; g.DB = s.sh;
	g.M = N * s.H * s.W; g.K = s.RH * s.RW * s.F; g.F = s.C;
	g.ldw = round_up(s.C, WT_COL_PAD);
	plain_output(g);
	return g;
}

/* The input gradient of a strided convolution, class by class. Input position a receives receptor row r only from
 * output row (a + pv - (dv + 1) r) / sv, if that divides: for the positions of one residue class a = a0 (mod sv) these are
 * the receptor rows r = r0 (mod sv), and with a = a0 + sv a', r = r0 + sv r' the output row is a' + PA - (dv + 1) r' - a
 * stride-1 gather over the sub-sampled receptor (likewise along the width). So sv * sh GEMMs without divisions, each with
 * only the taps that reach its positions, replace one GEMM over all taps of which 1 / (sv sh) are not zero; each writes
 * its class of positions through the output map. Needs gcd(dv + 1, sv) = gcd(dh + 1, sh) = 1 (r0 unique). */
struct StridedClass {
	int a0, b0, OAc, OBc, r0, s0, Rc, Sc, PA, PB;
	size_t wt_offset;       /* of the class's prepared weights in the buffer, in elements */
};

int gcd_int(int a, int b) {
	while (b) {
		const int t = a % b;
		a = b;
		b = t;
	}
	return a;
}

bool strided_classes(const ConvShape& s, std::vector<StridedClass>* out, size_t* wt_elems) {
	if ((s.sv == 1 && s.sh == 1) || gcd_int(s.dv + 1, s.sv) != 1 || gcd_int(s.dh + 1, s.sh) != 1)
		return false;
	size_t total = 0;
	for (int b0 = 0; b0 < s.sh; ++b0)
		for (int a0 = 0; a0 < s.sv; ++a0) {
			StridedClass c;
			c.a0 = a0;
			c.b0 = b0;
			c.OAc = a0 < s.H ? (s.H - a0 + s.sv - 1) / s.sv : 0;
			c.OBc = b0 < s.W ? (s.W - b0 + s.sh - 1) / s.sh : 0;
			c.r0 = c.s0 = 0;
			while (((s.dv + 1) * c.r0 - (a0 + s.pv)) % s.sv != 0)
				++c.r0;
			while (((s.dh + 1) * c.s0 - (b0 + s.ph)) % s.sh != 0)
				++c.s0;
			c.Rc = c.r0 < s.RH ? (s.RH - c.r0 + s.sv - 1) / s.sv : 0;
			c.Sc = c.s0 < s.RW ? (s.RW - c.s0 + s.sh - 1) / s.sh : 0;
			c.PA = (a0 + s.pv - (s.dv + 1) * c.r0) / s.sv;
			c.PB = (b0 + s.ph - (s.dh + 1) * c.s0) / s.sh;
			c.wt_offset = total;
			total += (size_t) round_up(std::max(1, c.Rc * c.Sc * s.F), WT_ROW_PAD) * round_up(s.C, WT_COL_PAD);
			if (out)
				out->push_back(c);
		}
	if (wt_elems)
		*wt_elems = total;
	return true;
}

/* Class by class pays once each class is a launch worth making: the GEMMs of a class do 1 / (sv sh) of the rows, so the
 * whole problem has to be a few launch overheads' worth of matrix work. Below that the single launch over all taps,
 * zeros included, is faster (or the kernel for a handful of output columns, which skips taps by predicate). */
bool use_strided_classes(const ConvShape& s, int N) {
	if (s.C <= FEW_COLUMNS || N % 4 != 0 || !strided_classes(s, nullptr, nullptr))
		return false;
	const double useful = 2.0 * N * s.OH() * s.OW() * (double) s.K() * s.F;
	return useful >= 2e8 * s.sv * s.sh;
}

void check_sizes(const ConvShape& s, int N) {
	CATTLE_HIP_REQUIRE(N > 0, "batch size must be positive");
	const double lim = 2147483647.0;
	const double in_elems = (double) N * s.H * s.W * s.C, out_elems = (double) N * s.OH() * s.OW() * s.F;
	CATTLE_HIP_REQUIRE(in_elems <= lim && out_elems <= lim, "tensor exceeds 2^31-1 elements");
	/* gather offsets are formed in 32-bit arithmetic relative to positions inside the padding */
	const double padded = (double) N * (s.H + 2.0 * s.pv + s.RH * (s.dv + 1.0)) * (s.W + 2.0 * s.ph + s.RW * (s.dh + 1.0)) *
			std::max(s.C, s.F);
	CATTLE_HIP_REQUIRE(padded <= lim, "padded tensor exceeds 2^31-1 elements");
	/* wgrad_kernel packs the displacements of a receptor position as two 16-bit fields */
	CATTLE_HIP_REQUIRE((double) s.RH * (s.dv + 1) < 32768.0 && (double) s.RW * (s.dh + 1) < 32768.0, "dilated receptor field too large");
}

/* Weight-gradient tile shapes (K rows x F columns of the gradient per block) and the split of M. */
constexpr int WGRAD_MC = 32;

template<typename T>
struct WgradVariant {
	int bk, bf, waves;
	int mc;                         /* rows of M per reduction chunk; above 32 only with 16-byte loads */
	void (*launch)(const T* x, const T* og, T* partials, T* bias_partials, const GatherGeom&, const WgradSplit&, bool vec,
			const WgradAct<T>* act);
	int (*blocks_per_cu)();         /* what the runtime says fits on a CU (registers and LDS) */
};

template<typename T, int WK, int WF, int TK, int TF, int MINW = 1, int MC = WGRAD_MC>
void launch_wgrad_variant(const T* x, const T* og, T* partials, T* bias_partials, const GatherGeom& g, const WgradSplit& plan,
		bool vec, const WgradAct<T>* act) {
	constexpr int VEC = GemmCfg<T>::VEC;
	dim3 block(64 * WK * WF), grid((unsigned) round_up(plan.tiles * plan.splits, 8));
	/* derivative on the negative side: p0 + p1 * y */
	T p0 = (T) 0, p1 = (T) 0;
	if (act && act->pool_inds && act->kind < 0) {
		p0 = (T) 1;             /* no activation behind the pool: slope one on either side */
	} else if (act) {
		CATTLE_HIP_REQUIRE(act_sign_coded(act->kind) && act->p >= (T) 0, "only a rectifier can be undone while the gradient is loaded");
		p0 = act->kind == ACT_RELU ? (T) 0 : act->p;
		p1 = act->kind == ACT_ELU ? (T) 1 : (T) 0;
	}
	if (act && act->pool_inds) {
		CATTLE_HIP_REQUIRE(vec && act->dz == nullptr, "the weight gradient from a pooled gradient needs 16-byte loads and forms no full-size gradient");
		wgrad_pooled_kernel<T, WK, WF, TK, TF, MC, VEC><<<grid, block, 0, stream()>>>(x, og, partials, bias_partials, g, plan, act->y, p0, p1,
				act->pool_inds, act->pool_sh_a, act->pool_sh_b);
	} else if (vec) {
		if (act)        /* the extra operand registers do not fit a register cap: MIN_WAVES 1 */
			wgrad_kernel<T, WK, WF, TK, TF, MC, VEC, 1, true><<<grid, block, 0, stream()>>>(x, og, partials, bias_partials, g, plan, act->y, act->dz, p0, p1);
		else
			wgrad_kernel<T, WK, WF, TK, TF, MC, VEC, MINW><<<grid, block, 0, stream()>>>(x, og, partials, bias_partials, g, plan, (const T*) nullptr, (T*) nullptr, (T) 0, (T) 0);
	} else {
		if constexpr (MC == WGRAD_MC) {
			if (act)
				wgrad_kernel<T, WK, WF, TK, TF, MC, 1, 1, true><<<grid, block, 0, stream()>>>(x, og, partials, bias_partials, g, plan, act->y, act->dz, p0, p1);
			else
				wgrad_kernel<T, WK, WF, TK, TF, MC, 1, 1><<<grid, block, 0, stream()>>>(x, og, partials, bias_partials, g, plan, (const T*) nullptr, (T*) nullptr, (T) 0, (T) 0);
		} else
			CATTLE_HIP_REQUIRE(false, "a weight-gradient variant with long chunks was planned for scalar loads");
	}
	CATTLE_HIP_CHECK(hipGetLastError());
}

template<typename T, int WK, int WF, int TK, int TF, int MINW = 1, int MC = WGRAD_MC>
int wgrad_variant_occupancy() {
	static int cached = 0;
	if (cached == 0) {
		int n = 0;
		CATTLE_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, wgrad_kernel<T, WK, WF, TK, TF, MC, GemmCfg<T>::VEC, MINW>,
				64 * WK * WF, 0));
		cached = std::max(1, n);
	}
	return cached;
}

template<typename T, int WK, int WF, int TK, int TF, int MINW = 1, int MC = WGRAD_MC>
WgradVariant<T> wgrad_variant() {
	WgradVariant<T> v;
	v.bk = WK * TK;
	v.bf = WF * TF;
	v.waves = WK * WF;
	v.mc = MC;
	v.launch = &launch_wgrad_variant<T, WK, WF, TK, TF, MINW, MC>;
	v.blocks_per_cu = &wgrad_variant_occupancy<T, WK, WF, TK, TF, MINW, MC>;
	return v;
}

template<typename T> struct WgradVariants;
template<> struct WgradVariants<float> {
	static constexpr int COUNT = 11, BASE = 7;      /* BASE: the variants with the standard chunk, which any problem may use */
	static constexpr int WIDE_CHUNKS = 10;          /* 64 x 64 with chunks of 128 rows */
	static const WgradVariant<float>* get() {
		static const WgradVariant<float> v[COUNT] = {
			wgrad_variant<float, 2, 4, 96, 32, 4>(),    /* 192 x 128, registers held to four waves per SIMD = two blocks per CU */
			wgrad_variant<float, 2, 2, 64, 64>(),       /* 128 x 128 */
			wgrad_variant<float, 1, 4, 96, 32>(),       /*  96 x 128: K = 288 (3 x 3 x 32 channels) without padding */
			wgrad_variant<float, 1, 4, 32, 32>(),       /*  32 x 128 */
			wgrad_variant<float, 1, 4, 64, 32>(),       /*  64 x 128 */
			wgrad_variant<float, 2, 2, 32, 32>(),       /*  64 x 64: few filters */
			wgrad_variant<float, 1, 1, 32, 32>(),       /*  32 x 32, one wave: the first layer of a network (K = 27, a few filters) */
			/* the same small tiles with longer chunks of M: fewer, larger rounds of loads for latency-bound problems */
			wgrad_variant<float, 1, 1, 32, 32, 1, 128>(),
			wgrad_variant<float, 1, 1, 32, 32, 1, 64>(),
			wgrad_variant<float, 2, 2, 32, 32, 1, 64>(),
			wgrad_variant<float, 2, 2, 32, 32, 1, 128>(),
		};
		return v;
	}
};
template<> struct WgradVariants<double> {
	static constexpr int COUNT = 4, BASE = 4, WIDE_CHUNKS = -1;
	static const WgradVariant<double>* get() {
		static const WgradVariant<double> v[COUNT] = {
			wgrad_variant<double, 2, 4, 48, 32>(),      /* 96 x 128 */
			wgrad_variant<double, 2, 4, 48, 16>(),      /* 96 x 64 */
			wgrad_variant<double, 2, 2, 32, 32>(),      /* 64 x 64 */
			wgrad_variant<double, 1, 4, 32, 16>(),      /* 32 x 64 */
		};
		return v;
	}
};

struct WgradPlan {
	int variant, ktiles, ftiles, splits, chunks_per_split, pixel_mode;
};

/* The tile shape with the least padding wins (on ties the earlier, larger one, which re-reads G less often, unless only
 * a later one fits a CU twice); the
 * M range is then cut into as many slices as fill the chip once (blocks = tiles * splits <= slots),
 * so that no block runs in a second, mostly idle round; the slots are what the runtime's occupancy query
 * reports for the variant. The plan depends on the shape and the build only, which keeps the summation
 * order, and with it the result, reproducible. */
template<typename T>
WgradPlan wgrad_plan(int M, int K, int F, int N, bool vec) {
	const WgradVariant<T>* vars = WgradVariants<T>::get();
	WgradPlan p;
	p.variant = 0;
	long best = -1;
	for (int i = 0; i < WgradVariants<T>::BASE; ++i) {
		const long padded = (long) round_up(K, vars[i].bk) * round_up(F, vars[i].bf);
		if (best < 0 || padded < best) {
			best = padded;
			p.variant = i;
		}
	}
	/* Among the shapes with that padding, the first of which a CU holds two blocks: alone on its CU a block has nothing
	 * to cover its barriers and load waits with (fp64 at config 4: the 96 x 128 tile, one block per CU at 160 registers,
	 * 2.17 ms; the 96 x 64 tile, two blocks, 1.98 ms although it reads the input twice as often). */
	if (vars[p.variant].blocks_per_cu() < 2)
		for (int i = 0; i < WgradVariants<T>::BASE; ++i)
			if ((long) round_up(K, vars[i].bk) * round_up(F, vars[i].bf) == best && vars[i].blocks_per_cu() >= 2) {
				p.variant = i;
				break;
			}
	const Tuning& tune = tuning();
	/* A short reduction (a dense layer: M is the batch size) cannot be cut into many slices, so the tiles must fill the
	 * chip: among the shapes with the least padding, the largest whose tiles times the possible slices reach half of
	 * the CUs, else the one with the most tiles. Two chunks per block then, not four: measured, a block's time is its
	 * chain of chunks (about a microsecond each at these sizes), which the second launch that adds the slices costs less than. */
	const bool short_m = (M + WGRAD_MC - 1) / WGRAD_MC <= 16;
	if (short_m) {
		const int max_splits = std::max(1, (M + WGRAD_MC - 1) / WGRAD_MC / 2);
		int pick = -1;
		long most = -1;
		for (int i = 0; i < WgradVariants<T>::BASE; ++i) {
			if ((long) round_up(K, vars[i].bk) * round_up(F, vars[i].bf) != best)
				continue;
			const long blocks = (long) ((K + vars[i].bk - 1) / vars[i].bk) * ((F + vars[i].bf - 1) / vars[i].bf) * max_splits;
			if (blocks >= device_shape().cus / 2) {
				pick = i;
				break;
			}
			if (blocks > most) {
				most = blocks;
				pick = i;
			}
		}
		if (pick >= 0)
			p.variant = pick;
	}
	/* Many one-wave tiles over a long M (config 3's second convolution: 9 x 2 tiles of 32 x 32, 32768 rows): four-wave
	 * 64 x 64 tiles with chunks of 128 rows load each operand row half as often and in longer runs; measured 35 -> 28 us
	 * with the reduce launch. Needs 16-byte loads, and for the walk by positions a batch that is a multiple of the chunk. */
	if (!short_m && vec && WgradVariants<T>::WIDE_CHUNKS >= 0 && vars[p.variant].waves == 1) {
		const WgradVariant<T>& w = vars[WgradVariants<T>::WIDE_CHUNKS];
		const long tiles = (long) ((K + vars[p.variant].bk - 1) / vars[p.variant].bk) * ((F + vars[p.variant].bf - 1) / vars[p.variant].bf);
		const long padded = (long) round_up(K, w.bk) * round_up(F, w.bf);
		if (tiles >= 16 && padded * 100 <= best * 115 && N % w.mc == 0)
			p.variant = WgradVariants<T>::WIDE_CHUNKS;
	}
	if (tune.wgrad_variant >= 0 && tune.wgrad_variant < WgradVariants<T>::COUNT && (vec || vars[tune.wgrad_variant].mc == WGRAD_MC))
		p.variant = tune.wgrad_variant;
	const WgradVariant<T>& v = vars[p.variant];
	p.ktiles = (K + v.bk - 1) / v.bk;
	p.ftiles = (F + v.bf - 1) / v.bf;
	/* at most three blocks of eight waves per CU; small blocks up to sixteen waves' worth */
	const int occ = std::max(1, std::min(v.blocks_per_cu(), std::max(3, 16 / v.waves)));
	const int slots = device_shape().cus * occ;
	const int tiles = p.ktiles * p.ftiles;
	const int chunks = (M + v.mc - 1) / v.mc;
	int want = std::max(1, slots / tiles);
	/* at least four chunks per block; two where the chunks are 128 rows long (measured on 32768 x 288 x 64: 128 slices of
	 * two chunks 49.9 us for the backward pass, 64 slices of four 53.0 us) */
	const int min_chunks = tune.wgrad_min_chunks > 0 ? tune.wgrad_min_chunks : (short_m || v.mc >= 128 ? 2 : 4);
	want = std::min(want, std::max(1, chunks / min_chunks));
	/* a short reduction whose tiles already give every CU a block is not cut: the slices of a large gradient cost more to
	 * write, read back and add than the shorter chains save (dense 4096 -> 1024 at batch 512: two slices of 16.8 MB,
	 * 50 us + 33 us for the launch that adds them) */
	if (short_m && tiles >= device_shape().cus)
		want = 1;
	if (tune.wgrad_splits > 0)
		want = std::min(tune.wgrad_splits, chunks);
	p.chunks_per_split = (chunks + want - 1) / want;
	p.splits = (chunks + p.chunks_per_split - 1) / p.chunks_per_split;
	/* pixel mode: slices are ranges of output positions (each at least one), walked sample block by
	 * sample block; needs chunks that do not straddle positions */
	const int positions = M / N;
	p.pixel_mode = N % v.mc == 0 && positions >= 2 && !tune.wgrad_linear;
	if (p.pixel_mode)
		p.splits = std::max(1, std::min(want, positions));
	return p;
}

} /* namespace */

int dgrad_weight_layout(const ConvShape& s, int N) {
	return use_strided_classes(s, N) ? 1 : 0;
}

int prepared_weight_row_length(int columns) {
	return round_up(columns, WT_COL_PAD);
}

template<typename T>
ConvWorkspace conv_workspace(const ConvShape& s, int N) {
	check_sizes(s, N);
	ConvWorkspace ws;
	ws.wt_fwd = (size_t) round_up(s.K(), WT_ROW_PAD) * round_up(s.F, WT_COL_PAD);
	ws.wt_dgrad = (size_t) round_up(s.RH * s.RW * s.F, WT_ROW_PAD) * round_up(s.C, WT_COL_PAD);
	size_t by_class = 0;
	if (strided_classes(s, nullptr, &by_class))
		ws.wt_dgrad = std::max(ws.wt_dgrad, by_class);      /* either layout, whichever conv_input_gradient takes at a batch size */
	const int M = N * s.OH() * s.OW();
	const WgradPlan p = wgrad_plan<T>(M, s.K(), s.F, N, true), q = wgrad_plan<T>(M, s.K(), s.F, N, false);
	ws.partials = (size_t) std::max(p.splits, q.splits) * ((size_t) s.K() * s.F + (size_t) s.F);
	return ws;
}

template<typename T>
void conv_forward(const ConvShape& s, int N, const T* x, const T* w, const T* b, T* out, T* wt, bool wt_ready, int x_batch) {
	check_sizes(s, std::max(N, x_batch));
	GatherGeom g = forward_geom(s, N);
	if (x_batch > 0)
		g.NS = x_batch;
	if (!wt_ready) {
		const int Kp = round_up(g.K, WT_ROW_PAD);
		const size_t count = (size_t) Kp * g.ldw;
		prep_fwd_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wt, g.K, g.F, Kp, g.ldw);
		CATTLE_HIP_CHECK(hipGetLastError());
	}
	launch_gather<T>(x, wt, b, out, g);
}

template<typename T>
bool conv_forward_lstm(const ConvShape& s, int N, const T* x, int x_batch, const T* w, const T* b, T* wt, bool wt_ready,
		const LstmForwardStep<T>& step) {
	check_sizes(s, std::max(N, x_batch));
	GatherGeom g = forward_geom(s, N);
	if (x_batch > 0)
		g.NS = x_batch;
	Epilogue<T> E = { 0, (T) 0, nullptr, nullptr, 1, 1, 1, 1, nullptr, step };
	/* the prepared columns depend on the tile width, which the launcher chooses */
	const std::function<void(int)> prepare = [&](int bf) {
		if (wt_ready)
			return;
		const int Kp = round_up(g.K, WT_ROW_PAD);
		const size_t count = (size_t) Kp * g.ldw;
		prep_fwd_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wt, g.K, g.F, Kp, g.ldw, bf / 4);
		CATTLE_HIP_CHECK(hipGetLastError());
	};
	return launch_gather<T>(x, wt, b, (T*) nullptr, g, nullptr, EPI_LSTM, &E, nullptr, nullptr, nullptr, &prepare);
}

template<typename T>
bool conv_forward_fused(const ConvShape& s, int N, const T* x, const T* w, const T* b, T* out, T* wt, bool wt_ready, int epi,
		const Epilogue<T>& E, int* mtiles) {
	check_sizes(s, N);
	const GatherGeom g = forward_geom(s, N);
	if (epi == EPI_POOL) {
		CATTLE_HIP_REQUIRE(E.prh > 0 && E.prw > 0 && g.OA % E.prh == 0 && g.OB % E.prw == 0 && E.OHp == g.OA / E.prh &&
				E.OWp == g.OB / E.prw && (E.inds != nullptr || E.pool_mean), "the pooling epilogue needs windows that tile the output");
	}
	if (epi == EPI_STATS)
		CATTLE_HIP_REQUIRE(E.stats != nullptr, "the moments epilogue needs a buffer for its partials");
	/* the prepared weights come first: they are valid afterwards whatever the answer is */
	if (!wt_ready) {
		const int Kp = round_up(g.K, WT_ROW_PAD);
		const size_t count = (size_t) Kp * g.ldw;
		prep_fwd_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wt, g.K, g.F, Kp, g.ldw);
		CATTLE_HIP_CHECK(hipGetLastError());
	}
	/* the staging pass deals threads over windows of at most a tile's positions */
	if (epi == EPI_POOL && E.prh * E.prw > 64)
		return false;
	/* it writes 16 bytes of consecutive samples at a time */
	if (epi == EPI_POOL && (((reinterpret_cast<uintptr_t>(E.inds) | reinterpret_cast<uintptr_t>(E.pre)) & 15) != 0))
		return false;
	return launch_gather<T>(x, wt, b, out, g, nullptr, epi, &E, mtiles);
}

size_t conv_stats_rows(const ConvShape& s, int N) {
	/* the shortest tile of either variant table has 64 rows */
	return ((size_t) N * s.OH() * s.OW() + 63) / 64;
}

void static_scratch_setup() {
	int dev = -1;
	CATTLE_HIP_CHECK(hipGetDevice(&dev));
	CATTLE_HIP_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "device index beyond what the static scratch table holds");
	if (g_scratch_ptr[dev])
		return;
	void* ptr = nullptr;
	CATTLE_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
	g_scratch_ptr[dev] = ptr;
}

size_t static_scratch_bytes() {
	return STATIC_SCRATCH_BYTES;
}

template<typename T>
void conv_forward_static(const ConvShape& s, int N, const T* x, const T* w, const T* b, T* out) {
	check_sizes(s, N);
	int dev = -1;
	CATTLE_HIP_CHECK(hipGetDevice(&dev));
	CATTLE_HIP_REQUIRE(dev >= 0 && dev < MAX_DEVICES && g_scratch_ptr[dev] != nullptr, "the static scratch buffer of this device is not set up");
	ScratchArena arena = { static_cast<char*>(g_scratch_ptr[dev]), STATIC_SCRATCH_BYTES, 0 };
	const GatherGeom g = forward_geom(s, N);
	const int Kp = round_up(g.K, WT_ROW_PAD);
	const size_t count = (size_t) Kp * g.ldw;
	T* wt = static_cast<T*>(arena.take(count * sizeof(T), "prepared weights"));
	prep_fwd_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wt, g.K, g.F, Kp, g.ldw);
	CATTLE_HIP_CHECK(hipGetLastError());
	launch_gather<T>(x, wt, b, out, g, &arena);
}

template<typename T>
void conv_weight_gradient_with(const ConvShape& s, int N, const T* x, const T* out_grad, T* wgrad, T* bgrad, T* partials,
		const WgradAct<T>* act, ReduceBatch<T>* deferred, const std::function<bool(WgradRider<T>&)>* elsewhere);
template<typename T>
bool conv_input_gradient_with(const ConvShape& s, int N, const T* w, const T* out_grad, T* in_grad, T* wt_dgrad, bool wt_ready,
		const LstmBackwardStep<T>* then, int og_batch, WgradRider<T>* rider);

template<typename T>
void conv_weight_gradient(const ConvShape& s, int N, const T* x, const T* out_grad, T* wgrad, T* bgrad, T* partials,
		const WgradAct<T>* act, ReduceBatch<T>* deferred) {
	conv_weight_gradient_with<T>(s, N, x, out_grad, wgrad, bgrad, partials, act, deferred, nullptr);
}

/* `elsewhere`, if given, is offered the kernel launch when it is one that can ride in another launch (WgradRider) and
 * says whether it ran it; the sums of the slices follow here either way. */
template<typename T>
void conv_weight_gradient_with(const ConvShape& s, int N, const T* x, const T* out_grad, T* wgrad, T* bgrad, T* partials,
		const WgradAct<T>* act, ReduceBatch<T>* deferred, const std::function<bool(WgradRider<T>&)>* elsewhere) {
	check_sizes(s, N);
	if (deferred)
		deferred->count = 0;
	const GatherGeom g = forward_geom(s, N);
	/* split-M partials, then a fixed-order reduction that accumulates */
	const bool vec = N % GemmCfg<T>::VEC == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
			(reinterpret_cast<uintptr_t>(out_grad) & 15) == 0 &&
			(!act || ((reinterpret_cast<uintptr_t>(act->y) & 15) == 0 && (reinterpret_cast<uintptr_t>(act->dz) & 15) == 0 &&
					(reinterpret_cast<uintptr_t>(act->pool_inds) & 15) == 0));
	WgradPlan p = wgrad_plan<T>(g.M, g.K, g.F, N, vec);
	const WgradVariant<T>& v = WgradVariants<T>::get()[p.variant];
	const size_t count = (size_t) g.K * g.F;
	/* up to four filters over a long M: no matrix tiles (few_filters_wgrad_kernel). Its blocks are four source channels
	 * by a slice of M; slices so that the chip holds four of its wavefronts per SIMD and a wavefront still walks four
	 * row vectors or more before it adds up its lanes - never more than the plan's, whose partials the caller has room for. */
	const int taps = g.R * g.S;
	const bool few_filters = !act && vec && g.F <= FEW_COLUMNS && taps <= 16 && (long) g.M * g.K >= (16L << 20);
	if (few_filters) {
		const int channel_blocks = (g.LC + 3) / 4, row_vectors = (g.M + 64 * GemmCfg<T>::VEC - 1) / (64 * GemmCfg<T>::VEC);
		p.splits = std::max(1, std::min(p.splits, std::min(device_shape().cus * 4 / channel_blocks, row_vectors / 4)));
	}
	T* bias_partials = partials + (size_t) p.splits * count;
	static_assert(WGRAD_MC == 32, "the chunk length gather_with_wgrad_kernel is built with");
	const bool can_ride = elsewhere != nullptr && std::is_same<T, float>::value && !act && vec && v.bk == 32 && v.bf == 32 &&
			v.waves == 1 && v.mc == WGRAD_MC;
	auto run = [&](T* to_w, T* to_b, const WgradSplit& how) {
		if (few_filters) {
			const dim3 grid((unsigned) ((g.LC + 3) / 4), (unsigned) how.splits);
			constexpr int V = GemmCfg<T>::VEC;
			if (taps <= 9 && g.F == 3)
				few_filters_wgrad_kernel<T, V, 9, 3><<<grid, 256, 0, stream()>>>(x, out_grad, to_w, to_b, g, how.splits, how.direct);
			else if (taps <= 9)
				few_filters_wgrad_kernel<T, V, 9, FEW_COLUMNS><<<grid, 256, 0, stream()>>>(x, out_grad, to_w, to_b, g, how.splits, how.direct);
			else if (g.F == 3)
				few_filters_wgrad_kernel<T, V, 16, 3><<<grid, 256, 0, stream()>>>(x, out_grad, to_w, to_b, g, how.splits, how.direct);
			else
				few_filters_wgrad_kernel<T, V, 16, FEW_COLUMNS><<<grid, 256, 0, stream()>>>(x, out_grad, to_w, to_b, g, how.splits, how.direct);
			CATTLE_HIP_CHECK(hipGetLastError());
			return;
		}
		if (can_ride) {
			WgradRider<T> rider = { x, out_grad, to_w, to_b, g, how, false };
			if ((*elsewhere)(rider))
				return;
		}
		v.launch(x, out_grad, to_w, to_b, g, how, vec, act);
	};
	if (p.splits == 1) {
		/* one slice: every block owns its tile of the gradient and adds to it directly, no second launch */
		const WgradSplit direct = { p.ktiles, p.ktiles * p.ftiles, 1, p.chunks_per_split, p.pixel_mode, 1 };
		run(wgrad, bgrad, direct);
		return;
	}
	const WgradSplit split = { p.ktiles, p.ktiles * p.ftiles, p.splits, p.chunks_per_split, p.pixel_mode, 0 };
	run(partials, bias_partials, split);
	/* a few thousand outputs cut into many partials: a wavefront per output; else 64 outputs per block, 16-byte loads
	 * where counts and alignment allow */
	constexpr int V = 16 / (int) sizeof(T);
	const size_t outputs = count + (bgrad ? (size_t) g.F : 0);
	const bool wide = outputs <= 8192 && p.splits >= 32;
	const bool vec_sum = count % V == 0 && g.F % V == 0 && (reinterpret_cast<uintptr_t>(partials) & 15) == 0;
	ReduceBatch<T> both;
	both.count = 0;
	both.e[both.count++] = ReduceEntry<T>{ partials, wgrad, count, p.splits, 0, wide, vec_sum };
	if (bgrad)
		both.e[both.count++] = ReduceEntry<T>{ bias_partials, bgrad, (size_t) g.F, p.splits, 0, wide, vec_sum };
	if (deferred) {
		/* the caller adds the partial sums to the gradients later, together with those of other layers */
		*deferred = both;
		return;
	}
	reduce_partials_many<T>(both);
}

template<typename T>
void reduce_partials_many(ReduceBatch<T> batch) {
	if (batch.count == 0)
		return;
	CATTLE_HIP_REQUIRE(batch.count <= REDUCE_BATCH, "too many matrices in one reduce launch");
	int blocks = 0;
	for (int i = 0; i < batch.count; ++i) {
		ReduceEntry<T>& q = batch.e[i];
		q.first_block = blocks;
		const size_t per = q.wide ? 4 : 64;
		const size_t need = ((q.count + per - 1) / per + 7) / 8 * 8;      /* whole groups of eight: a block's XCD is its number modulo 8 */
		CATTLE_HIP_REQUIRE(need + (size_t) blocks <= 2147483647u, "gradients too large for one reduce launch");
		blocks += (int) need;
	}
	if (blocks == 0)
		return;
	reduce_partials_many_kernel<T><<<(unsigned) blocks, 256, 0, stream()>>>(batch);
	CATTLE_HIP_CHECK(hipGetLastError());
}

template<typename T>
bool conv_input_gradient(const ConvShape& s, int N, const T* w, const T* out_grad, T* in_grad, T* wt_dgrad, bool wt_ready,
		const LstmBackwardStep<T>* then, int og_batch) {
	return conv_input_gradient_with<T>(s, N, w, out_grad, in_grad, wt_dgrad, wt_ready, then, og_batch, nullptr);
}

/* (`rider`: a small weight-gradient launch that may run inside this one, see WgradRider) */
template<typename T>
bool conv_input_gradient_with(const ConvShape& s, int N, const T* w, const T* out_grad, T* in_grad, T* wt_dgrad, bool wt_ready,
		const LstmBackwardStep<T>* then, int og_batch, WgradRider<T>* rider) {
	check_sizes(s, std::max(N, og_batch));
	if (then == nullptr && use_strided_classes(s, N)) {
		std::vector<StridedClass> classes;
		strided_classes(s, &classes, nullptr);
		const int ldw = round_up(s.C, WT_COL_PAD);
		bool empty_class = false;
		for (const StridedClass& c : classes)
			empty_class = empty_class || (c.Rc * c.Sc == 0 && c.OAc * c.OBc > 0);
		if (empty_class)        /* positions that no tap reaches (a receptor narrower than the stride) */
			device_zero_fill(in_grad, (size_t) N * s.H * s.W * s.C * sizeof(T));
		std::vector<GatherGeom> geoms;
		std::vector<const T*> weights;
		for (const StridedClass& c : classes) {
			if (c.OAc * c.OBc == 0 || c.Rc * c.Sc == 0)
				continue;
			T* wtc = wt_dgrad + c.wt_offset;
			const int Kc = c.Rc * c.Sc * s.F, Kp = round_up(Kc, WT_ROW_PAD);
			if (!wt_ready) {
				const size_t count = (size_t) Kp * ldw;
				prep_dgrad_class_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wtc, s.RH, s.RW, s.C, s.F,
						c.r0, s.sv, c.Rc, c.s0, s.sh, c.Sc, Kp, ldw);
				CATTLE_HIP_CHECK(hipGetLastError());
			}
			GatherGeom g;
			g.N = N; g.NS = og_batch > 0 ? og_batch : N; g.LH = s.OH(); g.LW = s.OW(); g.LC = s.F;
			g.OA = c.OAc; g.OB = c.OBc;
			g.R = c.Rc; g.S = c.Sc;
			g.SA = 1; g.SB = 1; g.RA = -(s.dv + 1); g.RB = -(s.dh + 1); g.PA = c.PA; g.PB = c.PB; g.DA = 1; g.DB = 1;
			g.M = N * c.OAc * c.OBc; g.K = Kc; g.F = s.C;
			g.ldw = ldw;
			g.out_a0 = c.a0; g.out_sa = s.sv; g.out_b0 = c.b0; g.out_sb = s.sh; g.out_OA = s.H; g.out_M = N * s.H * s.W;
			geoms.push_back(g);
			weights.push_back(wtc);
		}
		/* the classes with the longest reductions first: their blocks are the ones the launch ends with otherwise */
		std::vector<size_t> order(geoms.size());
		for (size_t i = 0; i < order.size(); ++i)
			order[i] = i;
		std::stable_sort(order.begin(), order.end(), [&](size_t x, size_t y) { return geoms[x].K > geoms[y].K; });
		std::vector<GatherGeom> sorted_geoms;
		std::vector<const T*> sorted_weights;
		for (size_t i : order) {
			sorted_geoms.push_back(geoms[i]);
			sorted_weights.push_back(weights[i]);
		}
		geoms.swap(sorted_geoms);
		weights.swap(sorted_weights);
		/* one launch over all classes where 16-byte loads are possible, else a launch per class */
		const bool vec = N % GemmCfg<T>::VEC == 0 && (og_batch <= 0 || og_batch % GemmCfg<T>::VEC == 0) &&
				(reinterpret_cast<uintptr_t>(out_grad) & 15) == 0;
		if (!vec || !launch_gather_classes<T>(out_grad, in_grad, geoms, weights))
			for (size_t i = 0; i < geoms.size(); ++i)
				launch_gather<T>(out_grad, weights[i], (const T*) nullptr, in_grad, geoms[i]);
		return false;
	}
	GatherGeom d = dgrad_geom(s, N);
	if (og_batch > 0)
		d.NS = og_batch;
	if (!wt_ready) {
		const int Kp = round_up(d.K, WT_ROW_PAD);
		const size_t count = (size_t) Kp * d.ldw;
		prep_dgrad_weights_kernel<T><<<(unsigned) ((count + 255) / 256), 256, 0, stream()>>>(w, wt_dgrad, s.RH * s.RW, s.C, s.F,
				Kp, d.ldw);
		CATTLE_HIP_CHECK(hipGetLastError());
	}
	bool then_done = false;
	launch_gather<T>(out_grad, wt_dgrad, (const T*) nullptr, in_grad, d, nullptr, EPI_NONE, nullptr, nullptr, then, &then_done, nullptr, rider);
	return then_done;
}

template<typename T>
void conv_backward(const ConvShape& s, int N, const T* x, const T* w, const T* out_grad, T* wgrad, T* bgrad,
		T* in_grad, T* wt_dgrad, bool wt_ready, T* partials, const WgradAct<T>* act, ReduceBatch<T>* deferred) {
	CATTLE_HIP_REQUIRE(!act || !in_grad || act->dz != nullptr, "the input gradient needs the gradient before the activation");
	/* Without an activation to undo, the two gradients wait for the same upstream gradient only: where the weight gradient
	 * is a launch of one-wavefront tiles, the input-gradient launch takes its blocks along. */
	bool in_grad_done = false;
	const std::function<bool(WgradRider<T>&)> with_input_gradient = [&](WgradRider<T>& rider) {
		conv_input_gradient_with<T>(s, N, w, out_grad, in_grad, wt_dgrad, wt_ready, nullptr, 0, &rider);
		in_grad_done = true;
		return rider.done;
	};
	conv_weight_gradient_with<T>(s, N, x, out_grad, wgrad, bgrad, partials, act, deferred, in_grad && !act ? &with_input_gradient : nullptr);
	if (in_grad && !in_grad_done)
		conv_input_gradient<T>(s, N, w, act ? (const T*) act->dz : out_grad, in_grad, wt_dgrad, wt_ready, nullptr, 0);
}

template ConvWorkspace conv_workspace<float>(const ConvShape&, int);
template ConvWorkspace conv_workspace<double>(const ConvShape&, int);
template void conv_forward<float>(const ConvShape&, int, const float*, const float*, const float*, float*, float*, bool, int);
template void conv_forward<double>(const ConvShape&, int, const double*, const double*, const double*, double*, double*, bool, int);
template bool conv_forward_fused<float>(const ConvShape&, int, const float*, const float*, const float*, float*, float*, bool, int,
		const Epilogue<float>&, int*);
template bool conv_forward_fused<double>(const ConvShape&, int, const double*, const double*, const double*, double*, double*, bool, int,
		const Epilogue<double>&, int*);
template bool conv_forward_lstm<float>(const ConvShape&, int, const float*, int, const float*, const float*, float*, bool,
		const LstmForwardStep<float>&);
template bool conv_forward_lstm<double>(const ConvShape&, int, const double*, int, const double*, const double*, double*, bool,
		const LstmForwardStep<double>&);
template void conv_forward_static<float>(const ConvShape&, int, const float*, const float*, const float*, float*);
template void conv_forward_static<double>(const ConvShape&, int, const double*, const double*, const double*, double*);
template void conv_backward<float>(const ConvShape&, int, const float*, const float*, const float*, float*, float*, float*,
		float*, bool, float*, const WgradAct<float>*, ReduceBatch<float>*);
template void conv_backward<double>(const ConvShape&, int, const double*, const double*, const double*, double*, double*,
		double*, double*, bool, double*, const WgradAct<double>*, ReduceBatch<double>*);
template void conv_weight_gradient<float>(const ConvShape&, int, const float*, const float*, float*, float*, float*,
		const WgradAct<float>*, ReduceBatch<float>*);
template void conv_weight_gradient<double>(const ConvShape&, int, const double*, const double*, double*, double*, double*,
		const WgradAct<double>*, ReduceBatch<double>*);
template void reduce_partials_many<float>(ReduceBatch<float>);
template void reduce_partials_many<double>(ReduceBatch<double>);
template bool conv_input_gradient<float>(const ConvShape&, int, const float*, const float*, float*, float*, bool,
		const LstmBackwardStep<float>*, int);
template bool conv_input_gradient<double>(const ConvShape&, int, const double*, const double*, double*, double*, bool,
		const LstmBackwardStep<double>*, int);

} /* namespace cattle_hip */
