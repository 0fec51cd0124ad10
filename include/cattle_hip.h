/*
 * cattle_hip.h — C ABI of libcattle_hip.so: MI355X (gfx950) kernels for C-ATTL3's kernel-layer
 * hot path behind the contract of cattle::Layer<Scalar,Rank>.
 *
 * A layer handle is the device-side twin of one cattle::Layer object: it owns the forward caches
 * the reference layer keeps, device copies of the layer's parameters and an accumulating gradient
 * buffer per parameter. Citations name the reference interface each entry point stands in for
 * (paths relative to the reference's C-ATTL3/ directory).
 *
 * Data layout: every tensor is the reference's column-major buffer whose index order is
 * (N, H, W, C): offset(n,h,w,c) = n + N*(h + H*(w + W*c)) (core/EigenProxy.hpp:43-64). Rank-1 and
 * rank-2 layers pass their data re-viewed as (N,H,1,1) / (N,H,W,1) exactly as the reference does
 * (layer/kernel/ConvKernelLayer.hpp:400-417, :494-508). Matrices are column-major.
 *
 * Every function returns CATTLE_HIP_OK or an error code; cattle_hip_last_error() then returns a
 * message for the calling thread. Calls are serialised internally, so distinct layers may be
 * driven from different host threads (neural_network/ParallelNeuralNetwork.hpp:158-171); a single
 * layer is not re-entrant, as in the reference. No entry point falls back to host computation: if
 * no MI355X is usable, cattle_hip_init() fails and so does everything after it.
 */
#ifndef CATTLE_HIP_H_
#define CATTLE_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cattle_hip_layer_s* cattle_hip_layer_t;
typedef struct cattle_hip_timer_s* cattle_hip_timer_t;
typedef struct cattle_hip_graph_s* cattle_hip_graph_t;

enum {
	CATTLE_HIP_OK = 0,
	CATTLE_HIP_ERR_INVALID = 1,   /* bad argument or dimension mismatch (the reference asserts) */
	CATTLE_HIP_ERR_STATE = 2,     /* e.g. backward without a matching forward */
	CATTLE_HIP_ERR_DEVICE = 3,    /* HIP runtime failure */
	CATTLE_HIP_ERR_OOM = 4        /* device allocation failed */
};

/* Scalar of Layer<Scalar,Rank> (core/Layer.hpp:32). */
typedef enum { CATTLE_HIP_F32 = 0, CATTLE_HIP_F64 = 1 } cattle_hip_dtype;

/* Where a buffer argument lives. HOST buffers are pageable host memory (an Eigen tensor's data());
 * they are staged through device buffers owned by the layer. DEVICE buffers are used in place;
 * a DEVICE input that a layer caches for its backward pass (the layer input of conv, dense, ReLU,
 * ..., or the output of sigmoid/tanh) is borrowed, not copied: it must stay valid and unmodified
 * until the matching backward call or cattle_hip_layer_empty_cache(). */
typedef enum { CATTLE_HIP_HOST = 0, CATTLE_HIP_DEVICE = 1 } cattle_hip_memspace;

/* Activation layers of layer/activation/<Name>ActivationLayer.hpp. */
typedef enum {
	CATTLE_HIP_ACT_IDENTITY = 0, CATTLE_HIP_ACT_SCALED = 1, CATTLE_HIP_ACT_BINARY_STEP = 2,
	CATTLE_HIP_ACT_SIGMOID = 3, CATTLE_HIP_ACT_TANH = 4, CATTLE_HIP_ACT_SOFTSIGN = 5,
	CATTLE_HIP_ACT_SOFTPLUS = 6, CATTLE_HIP_ACT_RELU = 7, CATTLE_HIP_ACT_LEAKY_RELU = 8,
	CATTLE_HIP_ACT_ELU = 9, CATTLE_HIP_ACT_SWISH = 10, CATTLE_HIP_ACT_SOFTMAX = 11,
	CATTLE_HIP_ACT_PRELU = 12, CATTLE_HIP_ACT_PSWISH = 13
} cattle_hip_activation;

typedef enum { CATTLE_HIP_POOL_MAX = 0, CATTLE_HIP_POOL_MEAN = 1 } cattle_hip_pool;

/* ---- library ---------------------------------------------------------------------------- */

/* Selects the device and creates the library's stream. Fails unless the device is a gfx950. */
int cattle_hip_init(int device);
const char* cattle_hip_last_error(void);
/* Waits for all work issued by the library. */
int cattle_hip_synchronize(void);

/* Plain device memory for callers that keep activations resident between layers (the idea of
 * core/gpu/GPULayer.hpp:31-58: device-tensor overloads next to the host-tensor virtuals). */
int cattle_hip_alloc(void** device_ptr, size_t bytes);
/* Released blocks are kept by the library and handed out again (a hipFree would stall the device at every
 * layer of a step); cattle_hip_trim returns the idle ones to the driver. */
int cattle_hip_free(void* device_ptr);
int cattle_hip_trim(void);
/* Free and total memory of the device as the driver reports them (pooled idle buffers count as used). No counterpart
 * in the reference. */
int cattle_hip_memory_info(size_t* free_bytes, size_t* total_bytes);
int cattle_hip_upload(void* dst_device, const void* src_host, size_t bytes);
int cattle_hip_download(void* dst_host, const void* src_device, size_t bytes);
int cattle_hip_fill_zero(void* dst_device, size_t bytes);

/* Event timers on the library's stream (for benchmarks: kernel time with data resident). */
int cattle_hip_timer_create(cattle_hip_timer_t* timer);
int cattle_hip_timer_destroy(cattle_hip_timer_t timer);
int cattle_hip_timer_start(cattle_hip_timer_t timer);
int cattle_hip_timer_stop(cattle_hip_timer_t timer, float* elapsed_ms);   /* synchronises */

/* ---- layer construction ------------------------------------------------------------------ */

/* ---- recorded steps (no counterpart in the reference, whose training loop calls the layers anew for every batch:
 * optimizer/SGDOptimizer.hpp:44-70) -----------------------------------------------------------------------------------
 * Between cattle_hip_graph_begin_capture and cattle_hip_graph_end_capture the library's calls are recorded instead of
 * run: layer passes, loss gradients, optimizer steps on device-resident parameters, on DEVICE buffers only. What was
 * recorded runs, as one HIP graph, at every cattle_hip_graph_launch: a training step of twenty small kernels then costs
 * the host one call, which matters to a loop that reads the loss back after every batch. Rules:
 *  - run the same calls once, eagerly, first: buffers that a layer would have to allocate or grow, host copies, waits
 *    (cattle_hip_synchronize, _download, _layer_empty_cache, timers) return CATTLE_HIP_ERR_STATE while recording;
 *  - a launch repeats the recorded kernels with the recorded arguments: the same buffers (the caller's inputs, whatever
 *    cattle_hip_alloc returned during the recording; cattle_hip_free on them takes effect when the graph is destroyed),
 *    the same batch size, and the same scalars - an optimizer whose update depends on the time step or epoch (Adam,
 *    Nadam, AMSGrad, ...) is therefore called outside the recording, as is anything whose result the host must see;
 *  - a training pass of a dropout layer cannot be recorded (CATTLE_HIP_ERR_STATE): its mask is a function of the number
 *    of the pass, which a replay would not advance; record the layers on either side of it;
 *  - a graph holds the device addresses it was recorded with. As long as it exists, a buffer of the library that was
 *    allocated before the recording ended stays where it is: a call that would have to grow one (a layer that took
 *    part run at a larger batch size; any layer whose split reduction needs more of the shared scratch buffer than
 *    every call before the recording did) and cattle_hip_layer_empty_cache on a layer created before the recording
 *    return CATTLE_HIP_ERR_STATE until cattle_hip_graph_destroy; the buffers of a layer that is destroyed while the
 *    graph exists are kept until then, so that a later launch still finds memory of its own (its results are then
 *    meaningless, never a fault). Layers and buffers created after the recording are free to change;
 *  - layers that took part, and their caches, must be left alone while launches of the graph are in flight. */
int cattle_hip_graph_begin_capture(void);
int cattle_hip_graph_end_capture(cattle_hip_graph_t* graph);
int cattle_hip_graph_launch(cattle_hip_graph_t graph);
int cattle_hip_graph_destroy(cattle_hip_graph_t graph);

/* ConvKernelLayer<Scalar,Rank>(input_dims, filters, init, receptor_height, receptor_width,
 * vertical_padding, horizontal_padding, vertical_stride, horizontal_stride, vertical_dilation,
 * horizontal_dilation) — layer/kernel/ConvKernelLayer.hpp:282-296 (rank 2 :342-357, rank 1
 * :441-456). Dilation 0 means a dense receptor (:71-72). Parameters: 0 = weights
 * [receptor_height*receptor_width*channels x filters] with row index rh + RH*(rw + RW*c)
 * (:138-139), 1 = bias [1 x filters] (:48-55). */
int cattle_hip_conv_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, size_t filters,
		size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_stride, size_t horizontal_stride, size_t vertical_dilation, size_t horizontal_dilation,
		cattle_hip_layer_t* layer);

/* ConvKernelLayer::pass_forward without any allocation. No counterpart in the reference: it is for callers that cannot
 * allocate device memory while they call (code under HIP graph capture, tight serving loops, harnesses that forbid it).
 * It computes what cattle_hip_layer_forward computes for a layer made by cattle_hip_conv_create with the same geometry,
 * bit for bit, from buffers that the caller owns, all in device memory: `in_device` (batch, height, width, channels),
 * `weights_device` [receptor_height*receptor_width*channels x filters] in the layout of parameter 0, `bias_device`
 * [1 x filters] (NULL: no bias), `out_device` (batch, OH, OW, filters). Nothing is cached for a backward pass.
 * Its scratch memory (the re-laid-out weights and, for launches that cut reductions into parts, their partial sums) is
 * a fixed array inside the library, cattle_hip_static_scratch_bytes() bytes (72 MiB) per device, held from the moment the
 * library is loaded on a device until the process ends; a problem that needs more is refused with CATTLE_HIP_ERR_INVALID
 * and a message that names both sizes. Call cattle_hip_init() beforehand: the first call into the library creates its
 * stream. Every call on a device uses the same array, so calls that overlap on one device race: issue them from one
 * thread or serialise them (the library's own lock does; work that a caller issues outside the lock does not count). */
int cattle_hip_conv_forward_noalloc(cattle_hip_dtype dtype, size_t batch, size_t height, size_t width, size_t channels,
		size_t filters, size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_stride, size_t horizontal_stride, size_t vertical_dilation, size_t horizontal_dilation,
		const void* in_device, const void* weights_device, const void* bias_device, void* out_device);
int cattle_hip_static_scratch_bytes(size_t* bytes);

/* TransConvKernelLayer<Scalar,Rank>(input_dims, filters, init, receptor_height, receptor_width,
 * vertical_padding, horizontal_padding, vertical_stride, horizontal_stride, vertical_dilation,
 * horizontal_dilation) — layer/kernel/TransConvKernelLayer.hpp:285-299 (rank 2 :345-360, rank 1
 * :444-459). Output height = (height - 1) * stride + receptor + (receptor - 1) * dilation - 2 * padding
 * (:226-229). Parameters: 0 = weights [channels x receptor_height*receptor_width*filters] with column
 * index rh + RH*(rw + RW*f) (:46-48, :159-160), 1 = bias [1 x output volume], one entry per output
 * activation (:52-56, :172-173). */
int cattle_hip_transconv_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, size_t filters,
		size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_stride, size_t horizontal_stride, size_t vertical_dilation, size_t horizontal_dilation,
		cattle_hip_layer_t* layer);

/* DenseKernelLayer<Scalar,Rank>(input_dims, output_size, init) — layer/kernel/DenseKernelLayer.hpp:61-77.
 * input_volume = input_dims.get_volume(). Parameters: 0 = weights [input_volume x output_size],
 * 1 = bias [1 x output_size]. */
int cattle_hip_dense_create(cattle_hip_dtype dtype, size_t input_volume, size_t output_size, cattle_hip_layer_t* layer);

/* BatchNormLayer<Scalar,Rank,PerLastRank>(dims, norm_avg_decay, epsilon) — layer/BatchNormLayer.hpp:66-101
 * (per_last_rank != 0: one statistics group per channel) and :334-361 (per_last_rank == 0: one per
 * activation). Parameters, each [1 x groups]: 0 = running means, 1 = running inverse standard
 * deviations (both not optimizable), 2 = gammas, 3 = betas — the order of get_params() (:263-272,
 * :399-406); the per-channel reference layer holds them as `groups` separate 1x1 matrices. */
int cattle_hip_batchnorm_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, int per_last_rank,
		double norm_avg_decay, double epsilon, cattle_hip_layer_t* layer);
/* The avgs_init flag of the reference layer (BatchNormLayer.hpp:234-243): whether the running
 * statistics hold values yet. A fresh layer starts at 0; clones copy it. */
int cattle_hip_batchnorm_get_stats_initialized(cattle_hip_layer_t layer, int* initialized);
int cattle_hip_batchnorm_set_stats_initialized(cattle_hip_layer_t layer, int initialized);

/* <Name>ActivationLayer<Scalar,Rank>(dims[, param]) — layer/activation/<Name>ActivationLayer.hpp; volume =
 * dims.get_volume(). param is the scale (Scaled), alpha (LeakyReLU, ELU), beta (Swish), epsilon
 * (Softmax), or the initial alpha / beta of PReLU / PSwish, whose parameter 0 is [1 x volume]
 * (PReLUActivationLayer.hpp:62-65, PSwishActivationLayer.hpp:59-62); ignored otherwise. */
int cattle_hip_activation_create(cattle_hip_dtype dtype, cattle_hip_activation kind, size_t volume, double param,
		cattle_hip_layer_t* layer);

/* MaxPoolLayer / MeanPoolLayer<Scalar,Rank>(input_dims, receptor_height, receptor_width,
 * vertical_stride, horizontal_stride) — layer/pool/MaxPoolLayer.hpp:105-108,
 * layer/pool/MeanPoolLayer.hpp:62-65, geometry in layer/PoolLayer.hpp:53-76, :145-155. */
int cattle_hip_pool_create(cattle_hip_dtype dtype, cattle_hip_pool kind, size_t height, size_t width, size_t channels,
		size_t receptor_height, size_t receptor_width, size_t vertical_stride, size_t horizontal_stride,
		cattle_hip_layer_t* layer);

/* A kernel layer and the layers that a feed-forward network calls right after it, run as one layer. The reference
 * calls them one after another (neural_network/FeedforwardNeuralNetwork.hpp:112-127 forwards, :129-141 backwards: the
 * shape of test/gradient_test.cpp:585-592 and examples/cifar_convnet.cpp:24-41 is conv -> ReLU -> max pool); here
 * `layers` = { convolutional or dense layer [, batch norm] [, activation] [, pool] }, existing handles in call order, become
 * one handle whose pass_forward / pass_back (cattle_hip_layer_forward / _backward) equal those calls in sequence:
 * the activation (ActivationLayer.hpp:47-66 and the element-wise kinds above) is applied in the epilogue of the GEMM, max
 * pooling over windows that tile the output (MaxPoolLayer.hpp:38-80; stride = receptor) too, so that the full-size
 * activation tensor is never written, mean pooling over such windows likewise (MeanPoolLayer.hpp:35-47; what the
 * activation's derivative reads is then kept at every position, for the backward pass spreads the gradient over whole
 * windows), and the per-channel batch norm (BatchNormLayer.hpp:225-261) gets its moments from the GEMM's epilogue. The members keep their parameters (the fused handle lists them all, members' order, same objects),
 * the batch norm its running statistics, the max pool its arg-max cache (cattle_hip_maxpool_indices on the member).
 * Whatever cannot be fused (batch sizes without 16-byte rows, overlapping windows, softmax, PReLU, PSwish, per-activation
 * batch norm behind a convolution) runs as the members' own passes, still on the device. Rectifier outputs (ReLU,
 * LeakyReLU, ELU) carry the side of their input in the sign bit: -0 where a negative input was mapped to zero.
 * The members are borrowed: they must outlive the fused handle, and must not be called on their own between a fused
 * forward pass and its backward pass. A clone (cattle_hip_layer_clone) owns clones of the members. */
int cattle_hip_fused_create(const cattle_hip_layer_t* layers, size_t count, cattle_hip_layer_t* fused);
/* How the last forward pass of a fused handle ran: 0 none yet, 1 member by member, 2 activation in the GEMM epilogue,
 * 3 activation and max or mean pooling in the GEMM epilogue, 4 batch-norm moments from the GEMM epilogue + one chain pass. */
int cattle_hip_fused_last_mode(cattle_hip_layer_t fused, int* mode);

/* DropoutLayer<Scalar,Rank>(dims, dropout_prob, epsilon) - layer/DropoutLayer.hpp:33-42, passes :74-96: a training
 * pass multiplies by the inverted-dropout mask (0 where u <= dropout_prob, else 1 / (1 - dropout_prob + epsilon)), an
 * inference pass hands the input through, the backward pass multiplies the gradient by the mask of the last training
 * pass. The reference draws u from Eigen's generator; here u comes from splitmix64 keyed by `seed` and the number of
 * the training pass (bits per element as described in csrc/pointwise_kernels.hip), so runs are reproducible and the
 * mask need not be stored. Layers that must drop independently need different seeds. volume = dims.get_volume(). */
int cattle_hip_dropout_create(cattle_hip_dtype dtype, size_t volume, double dropout_prob, double epsilon, unsigned long long seed,
		cattle_hip_layer_t* layer);

/* ReshapeLayer<Scalar,Rank>(input_dims, output_dims) - layer/ReshapeLayer.hpp:31-39, passes :77-90. Dimensions as
 * (height, width, channels); lower ranks pad with ones. */
int cattle_hip_reshape_create(cattle_hip_dtype dtype, const size_t input_dims[3], const size_t output_dims[3],
		cattle_hip_layer_t* layer);

/* BroadcastLayer<Scalar,Rank>(input_dims, broadcast) - layer/BroadcastLayer.hpp:31-40, passes :69-101: the input
 * repeated broadcast[i] times along rank i; the backward pass sums the replicas rank by rank. */
int cattle_hip_broadcast_create(cattle_hip_dtype dtype, const size_t input_dims[3], const size_t broadcast[3],
		cattle_hip_layer_t* layer);

/* ---- the cattle::Layer contract (core/Layer.hpp:47-137) ------------------------------------- */

/* Layer::clone() (:47) when share_params == 0: deep copy including parameter values and gradients;
 * Layer::clone_with_shared_params() (:56) otherwise: the clone refers to the same device parameter
 * and gradient buffers (layer/KernelLayer.hpp:71-77). Forward caches are not copied. */
int cattle_hip_layer_clone(cattle_hip_layer_t layer, int share_params, cattle_hip_layer_t* clone);
int cattle_hip_layer_destroy(cattle_hip_layer_t layer);

/* Layer::get_input_dims() / get_output_dims() (:73, :80), always as (height, width, channels). */
int cattle_hip_layer_input_dims(cattle_hip_layer_t layer, size_t dims[3]);
int cattle_hip_layer_output_dims(cattle_hip_layer_t layer, size_t dims[3]);

/* Layer::is_input_layer() / set_input_layer() (:90, :96). An input layer skips the input gradient. */
int cattle_hip_layer_is_input_layer(cattle_hip_layer_t layer, int* is_input_layer);
int cattle_hip_layer_set_input_layer(cattle_hip_layer_t layer, int is_input_layer);

/* Layer::empty_cache() (:101). */
int cattle_hip_layer_empty_cache(cattle_hip_layer_t layer);

/* Layer::pass_forward(Data in, bool training) (:126). in holds batch * volume(input dims) scalars,
 * out receives batch * volume(output dims) scalars. */
int cattle_hip_layer_forward(cattle_hip_layer_t layer, const void* in, cattle_hip_memspace in_space, size_t batch,
		int training, void* out, cattle_hip_memspace out_space);

/* Layer::pass_back(Data out_grad) (:137). Must follow a forward call with the same batch size.
 * Parameter gradients ACCUMULATE into the layer's gradient buffers, as Parameters::accumulate_grad
 * does (parameters/StandardParameters.hpp:115-123). in_grad may be NULL exactly when the layer is
 * an input layer (the reference then returns a null tensor); it is never written in that case.
 * Exception kept from the reference: PReLU computes the input gradient even as an input layer
 * (PReLUActivationLayer.hpp:87-109), so it requires in_grad unless it is NULL by choice. */
int cattle_hip_layer_backward(cattle_hip_layer_t layer, const void* out_grad, cattle_hip_memspace grad_space, size_t batch,
		void* in_grad, cattle_hip_memspace in_grad_space);

/* ---- Parameters (core/Parameters.hpp:15-95) ------------------------------------------------- */

/* Layer::get_params().size() (core/Layer.hpp:107-113). */
int cattle_hip_layer_num_params(cattle_hip_layer_t layer, size_t* count);
/* Parameters::get_rows() / get_cols() / are_optimizable(). */
int cattle_hip_layer_param_shape(cattle_hip_layer_t layer, size_t index, size_t* rows, size_t* cols, int* optimizable);
/* Parameters::set_values(Matrix) / get_values(): column-major rows x cols scalars. */
int cattle_hip_layer_set_param_values(cattle_hip_layer_t layer, size_t index, const void* values, cattle_hip_memspace space);
int cattle_hip_layer_get_param_values(cattle_hip_layer_t layer, size_t index, void* values, cattle_hip_memspace space);
/* Parameters::get_grad(): the gradient accumulated by backward calls since the last reset. */
int cattle_hip_layer_get_param_grad(cattle_hip_layer_t layer, size_t index, void* grad, cattle_hip_memspace space);
/* Parameters::reset_grad(). */
int cattle_hip_layer_reset_param_grad(cattle_hip_layer_t layer, size_t index);

/* The argmax cache of MaxPoolLayer (layer/pool/MaxPoolLayer.hpp:58-62, :82): OH*OW rows of
 * channels*batch unsigned entries, row = ow*OH + oh, column = c*batch + n, value =
 * w_in_window*receptor_height + h_in_window. Valid after a forward call. */
int cattle_hip_maxpool_indices(cattle_hip_layer_t layer, unsigned* indices, cattle_hip_memspace space);

/* ---- Device-resident training step: losses and optimizer updates ------------------------------
 * With these a whole step (propagate, loss, backpropagate, update, reset) runs on buffers that
 * never leave HBM; only the per-sample losses come back if the caller asks for them. */

typedef enum cattle_hip_loss {
	CATTLE_HIP_LOSS_SQUARED = 0,                    /* loss/SquaredLoss.hpp:25-34 */
	CATTLE_HIP_LOSS_SOFTMAX_CROSS_ENTROPY = 1,      /* loss/SoftmaxCrossEntropyLoss.hpp:33-50 */
	CATTLE_HIP_LOSS_ABSOLUTE = 2,                   /* loss/AbsoluteLoss.hpp:25-35 */
	CATTLE_HIP_LOSS_BINARY_CROSS_ENTROPY = 3,       /* loss/BinaryCrossEntropyLoss.hpp:35-46; sample_size must be 1 */
	CATTLE_HIP_LOSS_CROSS_ENTROPY = 4,              /* loss/CrossEntropyLoss.hpp:33-42 */
	CATTLE_HIP_LOSS_KULLBACK_LEIBLER = 5,           /* loss/KullbackLeiblerLoss.hpp:32-43 */
	CATTLE_HIP_LOSS_HINGE = 6,                      /* loss/HingeLoss.hpp:31-99, Squared = false */
	CATTLE_HIP_LOSS_SQUARED_HINGE = 7,              /* loss/HingeLoss.hpp:31-99, Squared = true */
	CATTLE_HIP_LOSS_MULTI_LABEL_HINGE = 8,          /* loss/MultiLabelHingeLoss.hpp:31-71, Squared = false */
	CATTLE_HIP_LOSS_SQUARED_MULTI_LABEL_HINGE = 9,  /* loss/MultiLabelHingeLoss.hpp:31-71, Squared = true */
	CATTLE_HIP_LOSS_MULTI_LABEL_LOG = 10,           /* loss/MultiLabelLogLoss.hpp:37-76 */
	/* a flag to OR into one of the kinds above: the loss wrapped in NegatedLoss (loss/NegatedLoss.hpp:41-46),
	 * whose function and d_function are the wrapped loss's with the opposite sign */
	CATTLE_HIP_LOSS_NEGATED = 0x100
} cattle_hip_loss;

/* Loss::function (loss/UniversalLoss.hpp:37-41 non-sequential, :99-110 sequential): `losses`
 * receives one value per sample, summed over the time steps. `out` and `obj` are
 * (batch, time_steps, sample_size) column-major; pass time_steps = 1 for non-sequential data.
 * `epsilon` is the constructor argument of the losses that have one (the cross entropies, Kullback-Leibler,
 * multi-label log; ignored by the others). The hinge losses take one-hot objectives; a row without a one,
 * which the reference asserts against, gets NaN as its loss and gradient. */
int cattle_hip_loss_function(cattle_hip_dtype dtype, cattle_hip_loss kind, const void* out, cattle_hip_memspace out_space,
		const void* obj, cattle_hip_memspace obj_space, size_t batch, size_t time_steps, size_t sample_size,
		double epsilon, void* losses, cattle_hip_memspace losses_space);
/* Loss::d_function (loss/UniversalLoss.hpp:42-46, :111-125) times `scale`; scale = 1 / batch_size
 * is the division SGDOptimizer::_train applies before backpropagating (optimizer/SGDOptimizer.hpp:54-55).
 * `grad` has the shape of `out` and may alias it. */
int cattle_hip_loss_d_function(cattle_hip_dtype dtype, cattle_hip_loss kind, const void* out, cattle_hip_memspace out_space,
		const void* obj, cattle_hip_memspace obj_space, size_t batch, size_t time_steps, size_t sample_size,
		double epsilon, double scale, void* grad, cattle_hip_memspace grad_space);

/* The optimizers of the optimizer/ directory as in-place updates of one Parameters object on the device:
 * <Name>Optimizer::_update_params for parameter `index` of `layer`, with the constructor arguments of
 * the reference optimizer in `hyper` (unused entries are ignored):
 *   VANILLA_SGD            learning_rate                                   VanillaSGDOptimizer.hpp:30-43
 *   MOMENTUM_SGD           init_learning_rate, annealing_rate, momentum    MomentumSGDOptimizer.hpp:35-72
 *   NESTEROV_MOMENTUM_SGD  init_learning_rate, annealing_rate, momentum    NesterovMomentumSGDOptimizer.hpp:37-55
 *   ADAGRAD                learning_rate, epsilon                          AdaGradOptimizer.hpp:32-70
 *   RMSPROP                learning_rate, l2_decay, epsilon                RMSPropOptimizer.hpp:34-47
 *   ADADELTA               decay, epsilon                                  AdaDeltaOptimizer.hpp:33-67
 *   ADAM, ADAMAX, NADAM, AMSGRAD   learning_rate, l1_decay, l2_decay, epsilon
 *                          AdamOptimizer.hpp:40-82, AdaMaxOptimizer.hpp:39-60, NadamOptimizer.hpp:39-65, AMSGradOptimizer.hpp:39-66
 * `epoch` is the zero-based epoch index SGDOptimizer::_train passes on (optimizer/SGDOptimizer.hpp:64: epoch - 1),
 * used by the annealed learning rate; `timestep` the zero-based update count (:65-66), used by the bias corrections.
 * The optimizer's state matrices (accumulated gradients, moving averages; up to three) live with the parameter
 * on the device, start at zero and are shared between layers that share the parameter; switching optimizers
 * calls for cattle_hip_layer_param_reset_optimizer_state (the optimizer's _fit). */
typedef enum cattle_hip_optimizer {
	CATTLE_HIP_OPT_VANILLA_SGD = 0, CATTLE_HIP_OPT_MOMENTUM_SGD = 1, CATTLE_HIP_OPT_NESTEROV_MOMENTUM_SGD = 2,
	CATTLE_HIP_OPT_ADAGRAD = 3, CATTLE_HIP_OPT_RMSPROP = 4, CATTLE_HIP_OPT_ADADELTA = 5, CATTLE_HIP_OPT_ADAM = 6,
	CATTLE_HIP_OPT_ADAMAX = 7, CATTLE_HIP_OPT_NADAM = 8, CATTLE_HIP_OPT_AMSGRAD = 9
} cattle_hip_optimizer;
int cattle_hip_layer_param_optimizer_update(cattle_hip_layer_t layer, size_t index, cattle_hip_optimizer optimizer,
		const double hyper[4], size_t epoch, size_t timestep);
/* The same update followed by Parameters::reset_grad of that parameter, the order in which SGDOptimizer::_train
 * applies them to every batch (optimizer/SGDOptimizer.hpp:64, :68-70), as one kernel: the gradient is zeroed by
 * the thread that has just used it. */
int cattle_hip_layer_param_optimizer_step(cattle_hip_layer_t layer, size_t index, cattle_hip_optimizer optimizer,
		const double hyper[4], size_t epoch, size_t timestep);

/* The loop of SGDOptimizer::_train over the parameters of a network (optimizer/SGDOptimizer.hpp:64, :68-70) as one
 * launch per sixteen parameters: entry i names parameter indices[i] of layers[i]; each is updated as by
 * cattle_hip_layer_param_optimizer_step. A Parameters object shared by several listed layers is updated once (the
 * reference's get_all_unique_params, core/NeuralNetwork.hpp). All listed layers must have one scalar type. */
int cattle_hip_optimizer_step_many(const cattle_hip_layer_t* layers, const size_t* indices, size_t count,
		cattle_hip_optimizer optimizer, const double hyper[4], size_t epoch, size_t timestep);

/* VanillaSGDOptimizer::_update_params for one Parameters object (optimizer/VanillaSGDOptimizer.hpp:38-43):
 * values -= grad * learning_rate, in place on the device. Non-optimizable parameters are rejected. */
int cattle_hip_layer_param_sgd_update(cattle_hip_layer_t layer, size_t index, double learning_rate);
/* AdamOptimizer::_update_params for one Parameters object (optimizer/AdamOptimizer.hpp:66-82) with
 * the reference's bias corrections 1 / (1 - (1 - decay)^(timestep + 1) + epsilon) and epsilon inside
 * the square root. The two moving averages live with the parameter on the device (shared between
 * layers that share the parameter) and start at zero. */
int cattle_hip_layer_param_adam_update(cattle_hip_layer_t layer, size_t index, double learning_rate, double l1_decay,
		double l2_decay, double epsilon, size_t timestep);
/* The ParameterRegularization of a Parameters object (the `weight_reg` / `bias_reg` constructor arguments of the kernel
 * layers, parameters/StandardParameters.hpp:60-76): L1ParameterRegularization(lambda) = (lambda, 0),
 * L2ParameterRegularization(lambda) = (0, lambda), ElasticNetParameterRegularization(l1, l2) = (l1, l2), none = (0, 0)
 * (the headers of parameter_regularization/). cattle_hip_layer_param_optimizer_step and cattle_hip_optimizer_step_many then add
 * the regularization's d_function at the current values to the gradient before the update, as SGDOptimizer::_train
 * does through Parameters::regularize (optimizer/SGDOptimizer.hpp:59-63, StandardParameters.hpp:133-136);
 * cattle_hip_layer_param_optimizer_update, which is _update_params alone, does not. */
int cattle_hip_layer_param_set_regularization(cattle_hip_layer_t layer, size_t index, double l1_lambda, double l2_lambda);
/* The value and gradient constraints of a Parameters object (the weight_clip, weight_max_l1_norm, ... bias_grad_max_l2_norm
 * constructor arguments of the kernel layers, parameters/StandardParameters.hpp:61-76), for parameters that stay on the
 * device; 0 switches a limit off. As in the reference (:105-123, :150-182): the values are constrained whenever they are
 * set (cattle_hip_layer_set_param_values, every optimizer update), the gradient after every accumulation (every
 * cattle_hip_layer_backward of a layer that holds the parameter, and the regularization term of an optimizer step), each
 * time in the order clip to [-clip, clip], scale by max_l1 / norm() if the Euclidean norm - which is what the reference's
 * "L1" constraint measures - exceeds max_l1, scale by max_l2 / squaredNorm() if the squared norm exceeds max_l2. */
int cattle_hip_layer_param_set_constraints(cattle_hip_layer_t layer, size_t index, double value_clip, double value_max_l1_norm,
		double value_max_l2_norm, double grad_clip, double grad_max_l1_norm, double grad_max_l2_norm);
/* Parameters::get_regularization_penalty (StandardParameters.hpp:128-132): l1 * sum |v| + 0.5 * l2 * sum v^2, 0 for
 * parameters without regularization or that are not optimizable. */
int cattle_hip_layer_param_regularization_penalty(cattle_hip_layer_t layer, size_t index, double* penalty);

/* The optimizer's _fit (e.g. optimizer/AdamOptimizer.hpp:55-65): zero the state matrices. */
int cattle_hip_layer_param_reset_optimizer_state(cattle_hip_layer_t layer, size_t index);

/* ---- Convolutional LSTM with fused gates ------------------------------------------------------
 * LSTMNeuralNetwork<Scalar,3,MulInt,false> (neural_network/LSTMNeuralNetwork.hpp:27-120 constructor,
 * :236-403 propagate, :404-503 backpropagate; multiplicative integration by
 * cattle_hip_convlstm_set_multiplicative_integration; not stateful, not reversed) whose eight kernels are ConvKernelLayers with `hidden_channels` filters and one receptor
 * geometry that keeps the spatial dimensions (stride 1), and whose five activations are element-wise
 * kinds (CATTLE_HIP_ACT_IDENTITY .. CATTLE_HIP_ACT_SWISH) given in the order forget, write, candidate,
 * state, read with their scalar arguments (NULL = all zero). `foremost` as in the constructor (:81):
 * a foremost network computes no input gradient.
 *
 * The handle is a cattle_hip_layer_t: clone/destroy, the parameter entry points and the optimizer
 * updates work on it with FOUR fused parameters — 0: input-side weights
 * [receptor_height*receptor_width*channels x 4*hidden_channels], column blocks forget | write |
 * candidate | read; 1: input-side biases [1 x 4*hidden_channels]; 2, 3: the same for the
 * output-side (recurrent) kernels, [receptor_height*receptor_width*hidden_channels x 4*hidden_channels].
 * cattle_hip_layer_forward/backward are refused: sequences go through the two calls below. */
int cattle_hip_convlstm_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, size_t hidden_channels,
		size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_dilation, size_t horizontal_dilation, const int activation_kinds[5], const double activation_params[5],
		int foremost, cattle_hip_layer_t* lstm);
/* NeuralNetwork::propagate (:236-403). input is (batch, input_seq_length, height, width, channels), out
 * (batch, output_seq_length, height, width, hidden_channels), column-major (core/NeuralNetwork.hpp:26);
 * output_seq_length and output_seq_delay are what the network's OutputSeqSizeFunc returns for this input
 * length (:241-243). A DEVICE input is borrowed until the matching backpropagate. */
int cattle_hip_convlstm_propagate(cattle_hip_layer_t lstm, const void* input, cattle_hip_memspace input_space, size_t batch,
		size_t input_seq_length, size_t output_seq_length, size_t output_seq_delay, int training, void* out,
		cattle_hip_memspace out_space);
/* NeuralNetwork::backpropagate (:404-503): out_grad has the shape of out; in_grad the shape of input, and is
 * NULL exactly when the network is foremost. Kernel gradients accumulate. */
int cattle_hip_convlstm_backpropagate(cattle_hip_layer_t lstm, const void* out_grad, cattle_hip_memspace grad_space,
		void* in_grad, cattle_hip_memspace in_grad_space);
/* The parameters of one of the eight kernels in the order of get_layers() (:521-529): 0 input_forget,
 * 1 output_forget, 2 input_write, 3 output_write, 4 input_candidate, 5 output_candidate, 6 input_read,
 * 7 output_read; bias = 0 selects the weights [receptor volume x hidden_channels], 1 the bias
 * [1 x hidden_channels]: the kernel's block of columns of the fused parameter. */
int cattle_hip_convlstm_set_kernel_values(cattle_hip_layer_t lstm, size_t kernel, int bias, const void* values,
		cattle_hip_memspace space);
int cattle_hip_convlstm_get_kernel_values(cattle_hip_layer_t lstm, size_t kernel, int bias, void* values,
		cattle_hip_memspace space);
int cattle_hip_convlstm_get_kernel_grad(cattle_hip_layer_t lstm, size_t kernel, int bias, void* grad, cattle_hip_memspace space);
/* The MulInt template argument of LSTMNeuralNetwork (neural_network/LSTMNeuralNetwork.hpp:44): at a time step that has
 * both an input and a previous output, each gate's weighted input and weighted output are multiplied instead of added
 * (:303-311, :318-326, :334-342, :369-377; gradients :449-466). Off when the network is created. Changing it empties the
 * caches: propagate again before backpropagate. */
int cattle_hip_convlstm_set_multiplicative_integration(cattle_hip_layer_t lstm, int enabled);
/* How the last propagate and the last backpropagate ran (no counterpart in the reference; for tests and profiles): the
 * number of time steps whose element-wise part (gate activations and state update, :283-394; their backward, :436-466)
 * ran inside a kernel of the output-side convolutions instead of a kernel of its own - forward in the epilogue of the
 * convolution, backward in the kernel that sums the parts of the input gradient's reductions. Which steps can depends
 * on the shapes only (batch sizes with 16-byte rows, problems small enough for the short tiles, hidden sizes that are
 * multiples of 8 or 16, no multiplicative integration for the forward step); results are the same either way to
 * rounding. */
int cattle_hip_convlstm_fused_steps(cattle_hip_layer_t lstm, int* forward_steps, int* backward_steps);

#ifdef __cplusplus
}
#endif

#endif /* CATTLE_HIP_H_ */
