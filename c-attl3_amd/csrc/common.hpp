/*
 * common.hpp — shared declarations of the cattle_hip library internals (gfx950 only).
 */
#ifndef CATTLE_HIP_COMMON_HPP_
#define CATTLE_HIP_COMMON_HPP_

#include <hip/hip_runtime.h>
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

namespace cattle_hip {

/* Error carrier used inside the library; the C-ABI layer turns it into a status code plus the
 * thread-local message returned by cattle_hip_last_error(). */
struct Error : public std::runtime_error {
	int code;
	Error(int code, const std::string& what) : std::runtime_error(what), code(code) { }
};

enum { ERR_INVALID = 1, ERR_STATE = 2, ERR_DEVICE = 3, ERR_OOM = 4 };

#define CATTLE_HIP_CHECK(expr) do { \
	hipError_t _e = (expr); \
	if (_e != hipSuccess) \
		throw ::cattle_hip::Error(_e == hipErrorOutOfMemory ? ::cattle_hip::ERR_OOM : ::cattle_hip::ERR_DEVICE, \
				std::string(#expr) + ": " + hipGetErrorString(_e)); \
} while (0)

#define CATTLE_HIP_REQUIRE(cond, msg) do { \
	if (!(cond)) \
		throw ::cattle_hip::Error(::cattle_hip::ERR_INVALID, std::string(msg)); \
} while (0)

/* The stream every kernel and copy of the library is issued on. */
hipStream_t stream();
/* Whether that stream is recording a graph (between cattle_hip_graph_begin_capture and _end_capture). Work that cannot
 * be part of a graph - host copies, waits, allocations that replace a buffer - calls forbid_while_capturing. */
bool capturing();
void forbid_while_capturing(const char* what);

/* Allocations and recorded graphs share a clock: a device allocation made at alloc_clock_tick() is pinned while a graph
 * recorded later is alive (it may hold the address), and then must not be freed: its owner refuses to grow or release
 * it, or hands it to park_allocation, which frees it when the last such graph is destroyed. */
uint64_t alloc_clock_tick();
bool pinned_by_graph(uint64_t born);
void park_allocation(void* p, uint64_t born);

/* Copies between pageable host memory and the device on that stream; both return when the host buffer may be
 * reused (host_to_device) or holds the data (device_to_host). Large copies are staged through pinned buffers by
 * several host threads (CATTLE_HIP_COPY_THREADS, default 4; 0 leaves the staging to the runtime). */
void host_to_device(void* dst_dev, const void* src_host, size_t bytes);
void device_to_host(void* dst_host, const void* src_dev, size_t bytes);

/* Geometry of a gathered GEMM  out[M x F] = A[M x K] * Wt[K x F]  whose A matrix is never
 * materialised: A(m,k) is read from a column-major (N, LH, LW, LC) tensor.
 *   m = n + N*(a + OA*b)           k = r + R*(s + S*ch)
 *   ya = (a*SA + PA + r*RA) / DA   (must divide exactly and lie in [0, LH))
 *   yb = (b*SB + PB + s*RB) / DB   (must divide exactly and lie in [0, LW))
 *   A(m,k) = src[n + N*(ya + LH*(yb + LW*ch))], or 0 where the conditions fail (zero padding).
 * The forward convolution uses SA = stride, RA = dilation + 1, PA = -padding, DA = 1; the input
 * gradient uses SA = 1, RA = -(dilation + 1), PA = +padding, DA = stride on the output gradient. */
struct GatherGeom {
	int N, LH, LW, LC;
	int OA, OB;
	int R, S;
	int SA, SB, RA, RB, PA, PB, DA, DB;
	int M, K, F;
	int ldw;        /* row stride of the prepared weight matrix Wt (elements) */
	int NS;         /* samples between two positions of the gathered tensor: N, or more when the N samples are the
	                 * first of a larger batch (one time step of a sequence tensor (N, T, ...), whose step t starts
	                 * N t elements into it and has N T samples between positions) */
	/* Where row m = n + N (a + OA b), column f of the result goes: element n + N ((out_a0 + out_sa a) + out_OA (out_b0 +
	 * out_sb b)) + out_M f of `out`. Plain (0, 1, 0, 1, OA, M): out is the M x F matrix itself. Otherwise the rows are
	 * one residue class of the positions of a larger tensor (a strided input gradient computed class by class). */
	int out_a0, out_sa, out_b0, out_sb, out_OA, out_M;
};

/* Convolution hyper-parameters in the reference's terms (dilation 0 = dense receptor). */
struct ConvShape {
	int H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh;
	int OH() const { return (H - RH - (RH - 1) * dv + 2 * pv) / sv + 1; }
	int OW() const { return (W - RW - (RW - 1) * dh + 2 * ph) / sh + 1; }
	int K() const { return RH * RW * C; }
};

/* Sizes of the scratch buffers the GEMM launchers need for a batch of N (in elements of T). */
struct ConvWorkspace {
	size_t wt_fwd;      /* prepared forward weights  */
	size_t wt_dgrad;    /* prepared input-gradient weights */
	size_t partials;    /* split-M partial weight gradients + bias-gradient partials */
};

template<typename T> ConvWorkspace conv_workspace(const ConvShape& s, int N);
/* Row length of a prepared weight layout with `columns` used columns: wt_fwd is [rows][row length] over the F filters,
 * wt_dgrad over the C channels (rows zero-padded to whole reduction chunks, columns to the row length). */
int prepared_weight_row_length(int columns);

/* Forward: out(N,OH,OW,F) = conv(x; w) + b. w is the reference's [K x F] column-major matrix.
 * wt is scratch of conv_workspace().wt_fwd elements; if wt_ready is false it is (re)built from w.
 * x_batch > 0: x holds the first N of x_batch samples per position (GatherGeom::NS). */
template<typename T> void conv_forward(const ConvShape& s, int N, const T* x, const T* w, const T* b, T* out,
		T* wt, bool wt_ready, int x_batch = 0);

/* The same forward pass for callers that cannot allocate device memory: the prepared weights and the partial sums of a
 * split reduction live in a fixed device array of static_scratch_bytes() bytes per device, whose address
 * static_scratch_setup() looks up for the current device (once; called when the library is initialised). Throws
 * ERR_INVALID when the problem needs more scratch than that. Every call on a device uses the same array. */
void static_scratch_setup();
size_t static_scratch_bytes();
template<typename T> void conv_forward_static(const ConvShape& s, int N, const T* x, const T* w, const T* b, T* out);

/* An element-wise activation behind the kernel layer, undone while the weight gradient loads its G operand: out_grad is
 * then the gradient of the activation's output y (the coded output of a fused forward pass, act_math.hpp), the operand
 * is dz = act'(y) * out_grad, formed in registers on the way into LDS. dz, if not null, also receives it (written once,
 * by the blocks of the first k tile), for the input-gradient launch that follows. The rectifier family only (ReLU, LeakyReLU and ELU
 * with non-negative arguments), whose derivative is a function of the coded output's sign bit. */
template<typename T> struct WgradAct {
	const T* y;
	T* dz;
	int kind;
	T p;
	/* pool_inds != null: the gradient handed to the weight-gradient launch and `y` are the tensors behind a max pool
	 * whose windows of 2^pool_sh_a x 2^pool_sh_b (height x width, stride = receptor) tile the kernel layer's output, and
	 * pool_inds is the pool's arg-max cache; dz must be null (the full-size gradient is never formed in memory), the
	 * launch needs 16-byte loads, and kind may be -1 for no activation. */
	const unsigned* pool_inds;
	int pool_sh_a, pool_sh_b;
};
/* Partial sums that wait to be added to their gradients: entry e is `splits` matrices of `count` values each, one
 * after the other at `partials`, to be added to dst in the fixed order of reduce_partials_many (first_block is filled in
 * by it; wide / vec pick the form of the sum, set by whoever wrote the partials). */
constexpr int REDUCE_BATCH = 32;
template<typename T> struct ReduceEntry {
	const T* partials;
	T* dst;
	size_t count;
	int splits, first_block;
	bool wide, vec;
};
template<typename T> struct ReduceBatch { ReduceEntry<T> e[REDUCE_BATCH]; int count; };
/* dst += sum of the partials, for every entry, in one launch */
template<typename T> void reduce_partials_many(ReduceBatch<T> batch);

/* Backward: wgrad[K x F] += A^T G, bgrad[F] += colsum(G), in_grad = dgrad (skipped if null). With `act`, G is
 * act'(y) * out_grad (see WgradAct; act->dz must be given when in_grad is). With `deferred`, a weight gradient cut into
 * slices of M leaves the sum of its slices to the caller: the entries (none if the launch added to the gradients
 * itself) go to reduce_partials_many whenever the gradients are first needed, which spares a launch per layer. */
template<typename T> void conv_backward(const ConvShape& s, int N, const T* x, const T* w, const T* out_grad,
		T* wgrad, T* bgrad, T* in_grad, T* wt_dgrad, bool wt_ready, T* partials, const WgradAct<T>* act = nullptr,
		ReduceBatch<T>* deferred = nullptr);

/* The two halves of conv_backward on their own (the transposed convolution uses them with the roles
 * of input and output exchanged). bgrad may be null. */
template<typename T> void conv_weight_gradient(const ConvShape& s, int N, const T* x, const T* out_grad, T* wgrad, T* bgrad,
		T* partials, const WgradAct<T>* act = nullptr, ReduceBatch<T>* deferred = nullptr);
template<typename T> struct LstmBackwardStep;
/* og_batch > 0: out_grad holds the first N of og_batch samples per position (GatherGeom::NS). `then`, if given, is the LSTM backward step that consumes in_grad as the gradient of its hidden output: when the
 * launch cuts every tile's reduction into parts, the kernel that sums the parts runs the element-wise part of that
 * step on each sum instead of writing it. Returns whether it did; false: in_grad was written and the step is still to
 * be run (lstm_gates_backward). */
template<typename T> bool conv_input_gradient(const ConvShape& s, int N, const T* w, const T* out_grad, T* in_grad,
		T* wt_dgrad, bool wt_ready, const LstmBackwardStep<T>* then = nullptr, int og_batch = 0);
/* Which prepared layout conv_input_gradient builds in wt_dgrad at this batch size: 0 the plain one (all taps), 1 the
 * blocks of a strided convolution's residue classes. Prepared weights are current only for the layout they were built as. */
int dgrad_weight_layout(const ConvShape& s, int N);

/* Element-wise / reduction kernels (pointwise_kernels.hip). */
template<typename T> void act_forward(int kind, size_t n, T p, const T* x, T* y);
template<typename T> void act_backward(int kind, size_t n, T p, const T* x, const T* y, const T* g, T* dx);
template<typename T> void softmax_forward(int N, int V, T eps, const T* x, T* y);
template<typename T> void softmax_backward(int N, int V, const T* y, const T* g, T* dx);
template<typename T> void prelu_forward(int N, int V, const T* alpha, const T* x, T* y);
template<typename T> void prelu_backward(int N, int V, const T* alpha, const T* x, const T* g, T* alpha_grad, T* dx);
template<typename T> void pswish_forward(int N, int V, const T* beta, const T* x, T* y);
template<typename T> void pswish_backward(int N, int V, const T* beta, const T* x, const T* g, T* beta_grad, T* dx);

/* Batch norm over `groups` contiguous slabs of L elements (per-channel: slab = channel, L = N*H*W;
 * per-activation: slab = one activation's column, L = N). ws needs bn_workspace() elements. */
size_t bn_workspace(int groups, size_t L);
template<typename T> void bn_forward(int groups, size_t L, const T* x, const T* gamma, const T* beta, T* avg_mean,
		T* avg_inv_sd, bool stats_init, bool training, T decay, T eps, T* out, T* std_cache, T* inv_sd_cache, T* ws);
template<typename T> void bn_backward(int groups, size_t L, const T* out_grad, const T* gamma, const T* std_cache,
		const T* inv_sd_cache, T* gamma_grad, T* beta_grad, T* in_grad, T* ws);

struct PoolShape {
	int H, W, C, RH, RW, sv, sh;
	int OH() const { return (H - RH) / sv + 1; }
	int OW() const { return (W - RW) / sh + 1; }
};
template<typename T> void maxpool_forward(const PoolShape& s, int N, const T* x, T* out, unsigned* inds);
template<typename T> void maxpool_backward(const PoolShape& s, int N, const T* out_grad, const unsigned* inds, T* in_grad);
template<typename T> void meanpool_forward(const PoolShape& s, int N, const T* x, T* out);
template<typename T> void meanpool_backward(const PoolShape& s, int N, const T* out_grad, T* in_grad);

/* Zeroes `bytes` bytes (a multiple of 4, at a 4-byte aligned address) with a kernel on the library's stream. */
void device_zero_fill(void* dst, size_t bytes);
/* ---- fused kernel layer: convolution or dense -> [batch norm] -> [activation] -> [pool] --------------------------- */

/* The element-wise part of an LSTM cell step between the kernel layers. kind/param index: 0 forget,
 * 1 write, 2 candidate, 3 state, 4 read activation (element-wise kinds only). Per-step tensors hold
 * the four gates as consecutive blocks of P elements; `*_all` tensors are (N, T, ...) over all steps. */
template<typename T> struct LstmActs { int kind[5]; T param[5]; };
/* The tensors of one forward step: zx the weighted inputs of all steps (null at a step without input), z / gates /
 * state / act_state this step's slabs (z, the gates' pre-activation values, null when no gate activation's backward
 * pass reads its input), hprev_all the hidden outputs of all steps shifted by one (slab h_t receives this step's: it
 * is what the next step's output-side kernels read), out the network's output sequence (null at a step that emits
 * nothing). */
template<typename T> struct LstmForwardStep {
	LstmActs<T> a;
	int N;
	size_t P;
	const T* zx;
	int zx_T, zx_t;
	bool mul_int;
	const T* prev_state;
	T *z, *gates, *state, *act_state, *hprev_all;
	int h_T, h_t;
	T* out;
	int out_T, out_t;
};
/* The tensors of one backward step. dzh_all, the gate gradients of all steps as the output-side kernels receive them,
 * serves both their weight gradient at the end and, slab by slab, their input gradient. zx_fwd / zh_fwd: the step's weighted input (in the all-steps tensor) and weighted
 * previous output when the network integrates multiplicatively and the step had both; null otherwise. */
template<typename T> struct LstmBackwardStep {
	LstmActs<T> a;
	int N;
	size_t P;
	const T* out_grad;
	int og_T, og_t;
	const T *z, *gates, *prev_state, *state, *act_state;
	T *state_grad, *dzx_all;
	int x_T, x_t;
	T* dzh_all;
	int h_T, h_t;
	const T *zx_fwd, *zh_fwd;
};
/* What the gather GEMM does with a finished output tile besides adding the bias:
 *   EPI_NONE   out = acc + bias.
 *   EPI_ACT    out = activation(acc + bias) in the coded form of act_math.hpp; the pre-activation values go to `pre`
 *              when the activation's backward pass needs them.
 *   EPI_POOL   activation, then max pooling with windows that tile the output (stride = receptor): `out` is the pooled
 *              tensor, `inds` the arg-max cache in the layout of MaxPoolLayer (layer/pool/MaxPoolLayer.hpp:58-62), `pre`
 *              the pre-activation value at each arg-max (or null). Needs the blocked tile order with whole windows per tile.
 *              With pool_mean: mean pooling, see below.
 *   EPI_STATS  out = acc + bias, plus per tile and output column (count, mean, sum of squared deviations) of the tile's
 *              rows in `stats` [mtiles][F][3]: the batch-norm moments of the convolution output without reading it again.
 *   EPI_LSTM   the output columns are the four gates' weighted previous outputs of an LSTM cell; the element-wise part of
 *              the cell's forward step (`lstm`) runs on them and `out` is not written. The prepared weights' columns are
 *              then ordered so that a tile holds all four gates of its hidden channels (conv_forward_lstm). */
enum { EPI_NONE = 0, EPI_ACT = 1, EPI_POOL = 2, EPI_STATS = 3, EPI_LSTM = 4 };
template<typename T>
struct Epilogue {
	int kind;               /* cattle_hip_activation, element-wise kinds */
	T p;                    /* the activation's scalar argument */
	T* pre;
	unsigned* inds;
	int prh, prw;           /* pooling receptor (= stride) along height and width */
	int OHp, OWp;           /* pooled output extents */
	T* stats;
	LstmForwardStep<T> lstm;
	/* EPI_POOL with mean pooling (MeanPoolLayer.hpp:35-41) instead of max pooling: `out` is the mean of each window, taken
	 * in the window's width-major order, `inds` is unused, and `pre` is a tensor of the full, unpooled size that receives
	 * what the backward pass needs at every position: the pre-activation values if keep_input, else the coded outputs. */
	int pool_mean, keep_input;
};
/* conv_forward with a fused epilogue. Returns false, having launched nothing, when the problem does not allow the
 * epilogue (no 16-byte accesses, windows that do not fit the tiles): the caller then runs the layers one by one; the
 * prepared weights `wt` are valid afterwards either way.
 * `mtiles` receives the row count of the EPI_STATS partials; conv_stats_rows() bounds it for any launch. */
template<typename T> bool conv_forward_fused(const ConvShape& s, int N, const T* x, const T* w, const T* b, T* out, T* wt,
		bool wt_ready, int epi, const Epilogue<T>& E, int* mtiles);
size_t conv_stats_rows(const ConvShape& s, int N);
/* The output-side kernels of an LSTM cell step (s.F = 4 * hidden filters: forget | write | candidate | read) on the
 * previous hidden output x (the first N of x_batch samples per position if x_batch > 0), followed in the same kernel
 * by the element-wise part of the step: the weighted previous outputs never reach memory. `wt` (conv_workspace().wt_fwd
 * elements) is a prepared layout of its own, not the one conv_forward builds. Returns false, having launched nothing
 * and leaving wt alone, when the problem does not allow it (no 16-byte accesses, too many rows for the short tiles
 * that can stage a whole tile, a hidden size that does not fill tiles with whole gate groups). */
template<typename T> bool conv_forward_lstm(const ConvShape& s, int N, const T* x, int x_batch, const T* w, const T* b, T* wt,
		bool wt_ready, const LstmForwardStep<T>& step);
/* The layers behind the kernel layer, on its output z (N, H, W, C): element-wise activation `kind` (argument p) and a
 * pool (0 none, 1 max, 2 mean) whose prh x prw windows tile z exactly. */
struct ChainShape {
	int H, W, C, prh, prw, pool, kind;
	double p;
};
/* dz from the gradient g of the (pooled) output, the arg-max cache, and the coded output y or the pre-activation
 * values `pre` (both at the arg-max positions under max pooling, at every position under mean pooling or none) */
template<typename T> void chain_backward(const ChainShape& s, int N, const T* g, const unsigned* inds, const T* y, const T* pre, T* dz);
/* With a per-channel batch norm between kernel layer and activation: out = pool(act(bn(z))), the channel moments merged
 * from the GEMM epilogue's per-tile moments `stats` [mtiles][C][3] (training) or taken from the running statistics. */
size_t bn_chain_workspace(int channels);
template<typename T> void bn_chain_forward(const ChainShape& s, int N, int mtiles, bool training, bool stats_init, const T* z,
		const T* stats, const T* gamma, const T* beta, T* avg_mean, T* avg_inv_sd, T decay, T eps, T* mean_cache, T* inv_sd_cache,
		T* out, unsigned* inds);
template<typename T> void bn_chain_backward(const ChainShape& s, int N, const T* g, const unsigned* inds, const T* z, const T* gamma,
		const T* beta, const T* mean_cache, const T* inv_sd_cache, T* gamma_grad, T* beta_grad, T* dz, T* ws);

/* dst[i] += src[i] */
template<typename T> void axpy_one(size_t n, const T* src, T* dst);
/* dst[c + cols*r] (+)= src[r + rows*c] for a column-major rows x cols matrix src */
template<typename T> void transpose_matrix(int rows, int cols, const T* src, T* dst, bool accumulate);
/* x[n + N*e] += row[e]  (a 1 x V row vector added to every row of an N x V matrix) */
template<typename T> void add_row_vector(int N, size_t V, const T* row, T* x);
/* row[e] += sum_n x[n + N*e]  (column sums of an N x V matrix, accumulated) */
template<typename T> void accumulate_column_sums(int N, size_t V, const T* x, T* row);

/* DropoutLayer: y = x * mask(u) with the uniform numbers u regenerated from `key` (the key of training pass `pass` of a
 * layer seeded with `seed` is dropout_pass_key(seed, pass)); used for the forward and the backward pass. */
unsigned long long dropout_pass_key(unsigned long long seed, unsigned long long pass);
template<typename T> void dropout_apply(size_t n, unsigned long long key, T prob, T eps, const T* x, T* y);
/* BroadcastLayer on (N, H, W, C) -> (N, H bh, W bw, C bc) and the sum of the replicas back. */
template<typename T> void broadcast_forward(int H, int W, int C, int bh, int bw, int bc, int N, const T* x, T* out);
template<typename T> void broadcast_backward(int H, int W, int C, int bh, int bw, int bc, int N, const T* out_grad, T* in_grad);

/* zh: the step's weighted previous output (four gate blocks of P elements), null at the first step */
template<typename T> void lstm_gates_forward(const LstmForwardStep<T>& step, const T* zh);
/* dh: the gradient of the hidden output that came back from the step after, null at the last step */
template<typename T> void lstm_gates_backward(const LstmBackwardStep<T>& step, const T* dh);

/* Losses and optimizer updates (train_kernels.hip). A batch is N samples x T_steps x V elements,
 * column-major with the sample index fastest. */
enum { LOSS_SQUARED = 0, LOSS_SOFTMAX_CROSS_ENTROPY = 1, LOSS_ABSOLUTE = 2, LOSS_BINARY_CROSS_ENTROPY = 3, LOSS_CROSS_ENTROPY = 4,
	LOSS_KULLBACK_LEIBLER = 5, LOSS_HINGE = 6, LOSS_SQUARED_HINGE = 7, LOSS_MULTI_LABEL_HINGE = 8,
	LOSS_SQUARED_MULTI_LABEL_HINGE = 9, LOSS_MULTI_LABEL_LOG = 10, LOSS_KINDS = 11, LOSS_NEGATED = 0x100 };
template<typename T> void loss_function(int kind, int N, int T_steps, int V, T eps, const T* out, const T* obj, T* losses);
template<typename T> void loss_d_function(int kind, int N, int T_steps, int V, T eps, T scale, const T* out, const T* obj,
		T* grad);
/* Optimizer update rules; values equal cattle_hip_optimizer. hyper holds the constructor arguments of the
 * reference optimizer in their order (learning rates, decays, epsilon; unused entries ignored). */
enum { OPT_VANILLA_SGD = 0, OPT_MOMENTUM_SGD = 1, OPT_NESTEROV = 2, OPT_ADAGRAD = 3, OPT_RMSPROP = 4, OPT_ADADELTA = 5,
	OPT_ADAM = 6, OPT_ADAMAX = 7, OPT_NADAM = 8, OPT_AMSGRAD = 9 };
template<typename T> struct OptCoef { T c[8]; };
int optimizer_state_count(int rule);
/* One parameter of a multi-parameter optimizer launch: its n elements, gradient, values and state matrices, and,
 * for a K x F convolution or dense weight matrix whose prepared layouts are current, those layouts (wt_fwd with row
 * length ldw_fwd; wt_dgrad for a receptor of RHW positions with row length ldw_dgrad), else null. */
constexpr int OPT_BATCH = 16;
template<typename T> struct OptParam {
	T* grad; T* values; T* s0; T* s1; T* s2; T* wt_fwd; T* wt_dgrad;
	size_t n;
	int K, RHW, ldw_fwd, ldw_dgrad;
	T l1, l2;           /* the lambdas of the parameter's regularization (both 0: none) */
	/* `splits` partial sums of the gradient, n values each, that still wait to be added to it (a weight gradient cut
	 * into a few slices): the kernel adds them in ascending order, as reduce_partials_many would have; null: none */
	const T* parts;
	int splits;
};
/* how many partial sums an optimizer launch takes along per parameter (more go through reduce_partials_many first) */
constexpr int OPT_MAX_PARTS = 8;
template<typename T> struct OptBatch { OptParam<T> p[OPT_BATCH]; int count; };
/* update + gradient reset of every parameter of the batch, one launch */
template<typename T> void optimizer_step_many(int rule, const double hyper[4], size_t epoch, size_t timestep, const OptBatch<T>& batch);
/* reset_grad: zero the gradient in the same kernel, after it has been used */
/* l1, l2: the lambdas of the parameter's regularization, whose gradient is added before the update (both 0: none) */
template<typename T> void optimizer_update(int rule, const double hyper[4], size_t epoch, size_t timestep, size_t n,
		T* grad, T* s0, T* s1, T* s2, T* values, bool reset_grad, T l1, T l2);
/* sums[0] = sum |v|, sums[1] = sum v^2 over a parameter's n values (device pointers) */
template<typename T> void regularization_sums(size_t n, const T* values, T* sums);
/* The clip, "L1" and "L2" norm constraints of StandardParameters (:150-182) on a matrix of n values, in that order; a
 * limit of zero is off. */
template<typename T> void constrain_matrix(size_t n, T* m, double clip, double max_l1, double max_l2);
/* grad += the regularization's d_function at the values (Parameters::regularize) */
template<typename T> void add_regularization(size_t n, const T* values, T* grad, T l1, T l2);

} /* namespace cattle_hip */

#endif /* CATTLE_HIP_COMMON_HPP_ */
