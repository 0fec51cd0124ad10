/*
 * layers.hip — layer objects behind the C ABI declared in include/cattle_hip.h.
 *
 * Each handle mirrors one cattle::Layer object (core/Layer.hpp:30-155): it keeps what the
 * reference layer caches between pass_forward and pass_back, device copies of the parameters and
 * accumulating gradient buffers, and forwards the arithmetic to the kernels in gemm_kernels.hip
 * and pointwise_kernels.hip. There is no host implementation of any operation here.
 */
#include "common.hpp"
#include "act_math.hpp"
#include "../../include/cattle_hip.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

namespace cattle_hip {

namespace {

std::recursive_mutex g_mutex;
thread_local std::string g_last_error;
bool g_ready = false;
hipStream_t g_stream = nullptr;
bool g_capturing = false;

void ensure_init(int device) {
	if (g_ready)
		return;
	int count = 0;
	hipError_t e = hipGetDeviceCount(&count);
	if (e != hipSuccess || count <= 0)
		throw Error(ERR_DEVICE, "no HIP device is available; cattle_hip has no host fallback");
	CATTLE_HIP_REQUIRE(device >= 0 && device < count, "device index out of range");
	CATTLE_HIP_CHECK(hipSetDevice(device));
	hipDeviceProp_t prop;
	CATTLE_HIP_CHECK(hipGetDeviceProperties(&prop, device));
	if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
		throw Error(ERR_DEVICE, std::string("cattle_hip is built for gfx950 only, found ") + prop.gcnArchName);
	CATTLE_HIP_CHECK(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
	static_scratch_setup();
	g_ready = true;
}

/* Recorded graphs keep the device addresses of the buffers their kernels were given. A clock that ticks at every
 * allocation and at the end of every recording orders the two: an allocation made before the newest recording that
 * is still alive may be what that graph points into, so it must neither move nor go back to the driver until the
 * graph is destroyed. Growing or releasing such a buffer is refused (ERR_STATE); one whose owner is destroyed is
 * parked and freed when no living graph is older than it. */
uint64_t g_alloc_clock = 0;
std::vector<uint64_t> g_live_graphs;           /* clock values at which the living graphs were recorded */
struct Parked { void* p; uint64_t born; };
std::vector<Parked> g_parked;

uint64_t newest_live_graph() {
	uint64_t newest = 0;
	for (uint64_t at : g_live_graphs)
		newest = std::max(newest, at);
	return newest;
}

void free_unpinned_parked() {
	const uint64_t newest = newest_live_graph();
	size_t kept = 0;
	for (size_t i = 0; i < g_parked.size(); ++i) {
		if (g_parked[i].born < newest)
			g_parked[kept++] = g_parked[i];
		else
			(void) hipFree(g_parked[i].p);
	}
	g_parked.resize(kept);
}

/* Grow-only device buffer. */
struct DevBuf {
	void* p = nullptr;
	size_t cap = 0;
	uint64_t born = 0;
	DevBuf() { }
	DevBuf(const DevBuf&) = delete;
	DevBuf& operator=(const DevBuf&) = delete;
	~DevBuf() {
		/* the owner goes away: what a living graph may still point into waits for that graph's end */
		if (p && pinned_by_graph(born))
			park_allocation(p, born);
		else if (p)
			(void) hipFree(p);
	}
	bool pinned() const {
		return p != nullptr && pinned_by_graph(born);
	}
	void release() {
		if (pinned())
			throw Error(ERR_STATE, "a recorded graph may point into this buffer: destroy the graph (cattle_hip_graph_destroy) before releasing it");
		if (p)
			(void) hipFree(p);
		p = nullptr;
		cap = 0;
	}
	void* ensure(size_t bytes) {
		if (bytes > cap) {
			/* recorded work may already point into the old buffer */
			forbid_while_capturing("growing a buffer of a layer (run the step once, at this batch size, before recording it)");
			if (pinned())
				throw Error(ERR_STATE, "a recorded graph may point into a buffer that this call has to grow: destroy the graph "
						"(cattle_hip_graph_destroy) first, or run at the largest size before recording");
			release();
			const size_t want = (bytes + 255) / 256 * 256;
			CATTLE_HIP_CHECK(hipMalloc(&p, want));
			cap = want;
			born = alloc_clock_tick();
		}
		return p;
	}
};

void copy_in(void* dst_dev, const void* src, int space, size_t bytes) {
	if (bytes == 0)
		return;
	if (space == CATTLE_HIP_HOST)
		host_to_device(dst_dev, src, bytes);
	else
		CATTLE_HIP_CHECK(hipMemcpyAsync(dst_dev, src, bytes, hipMemcpyDeviceToDevice, stream()));
}

void copy_out(void* dst, int space, const void* src_dev, size_t bytes) {
	if (bytes == 0)
		return;
	if (space == CATTLE_HIP_HOST)
		device_to_host(dst, src_dev, bytes);
	else
		CATTLE_HIP_CHECK(hipMemcpyAsync(dst, src_dev, bytes, hipMemcpyDeviceToDevice, stream()));
}

void fill_zero(void* dst_dev, size_t bytes) {
	if (bytes == 0)
		return;
	/* every buffer of the library is made of 4- or 8-byte scalars and is zeroed by a kernel, which a caller may record
	 * into a graph; only an odd-sized caller buffer goes to the runtime's memset */
	if ((reinterpret_cast<uintptr_t>(dst_dev) & 3) == 0 && bytes % 4 == 0) {
		device_zero_fill(dst_dev, bytes);
	} else {
		forbid_while_capturing("zeroing a buffer that is not made of 4-byte words");
		CATTLE_HIP_CHECK(hipMemsetAsync(dst_dev, 0, bytes, stream()));
	}
}

/* Device memory handed out through cattle_hip_alloc. Activations of a training step are allocated and
 * released at every layer call; hipMalloc / hipFree would synchronise the device each time, so released
 * blocks are kept, by size class, and handed out again. Everything the library does is ordered on one
 * stream, so a block may be reused as soon as it has been given back: work that still reads it was issued
 * earlier on that stream. Blocks return to the driver in trim() or at process exit. */
struct DevicePool {
	std::map<size_t, std::vector<void*>> idle;      /* size class -> blocks */
	std::map<void*, size_t> live;                    /* block -> size class */
	std::map<const char*, size_t> idle_index;        /* idle block -> size class, for released() */
	size_t idle_bytes = 0;
	static size_t size_class(size_t bytes) {
		/* powers of two up to 1 MiB, then multiples of 1 MiB: at most 2x / ~0 % over-allocation */
		size_t c = 256;
		while (c < bytes && c < (1u << 20))
			c <<= 1;
		return c >= bytes ? c : (bytes + (1u << 20) - 1) / (1u << 20) * (1u << 20);
	}
	void* take(size_t bytes) {
		const size_t c = size_class(bytes ? bytes : 1);
		std::vector<void*>& bucket = idle[c];
		void* p = nullptr;
		if (!bucket.empty()) {
			p = bucket.back();
			bucket.pop_back();
			idle_index.erase(static_cast<const char*>(p));
			idle_bytes -= c;
		} else {
			hipError_t e = hipMalloc(&p, c);
			if (e == hipErrorOutOfMemory && idle_bytes > 0 && !g_capturing) {       /* give the idle blocks back and try again */
				(void) hipGetLastError();
				(void) hipStreamSynchronize(stream());
				trim();
				e = hipMalloc(&p, c);
			}
			CATTLE_HIP_CHECK(e);
		}
		live[p] = c;
		if (g_capturing)
			taken.push_back(p);
		return p;
	}
	/* the end of a graph: its blocks become ordinary ones again, the freed ones idle */
	void release_graph(std::vector<void*>* blocks) {
		for (std::map<void*, std::vector<void*>*>::iterator it = owner.begin(); it != owner.end();) {
			if (it->second == blocks)
				it = owner.erase(it);
			else
				++it;
		}
		std::vector<void*> freed;
		freed.swap(*blocks);
		for (void* b : freed)
			give_back(b);
	}
	/* Blocks that recorded kernels read and write at every launch of their graph must not be handed out again while
	 * the graph exists: those freed during a recording wait in `held` for the graph object, and those taken during a
	 * recording (`taken`, then `owner`) go to their graph, not to the idle lists, when they are freed later. */
	std::vector<void*> held, taken;
	std::map<void*, std::vector<void*>*> owner;
	void give_back(void* p) {
		std::map<void*, size_t>::iterator it = live.find(p);
		CATTLE_HIP_REQUIRE(it != live.end(), "cattle_hip_free of a pointer that cattle_hip_alloc did not return");
		if (g_capturing) {
			if (std::find(held.begin(), held.end(), p) == held.end())
				held.push_back(p);
			return;
		}
		std::map<void*, std::vector<void*>*>::iterator own = owner.find(p);
		if (own != owner.end()) {
			if (std::find(own->second->begin(), own->second->end(), p) == own->second->end())
				own->second->push_back(p);
			return;
		}
		idle[it->second].push_back(p);
		idle_index[static_cast<const char*>(p)] = it->second;
		idle_bytes += it->second;
		live.erase(it);
	}
	/* whether p points into a block that was handed out and has been given back since */
	bool released(const void* p) const {
		if (!p || idle_index.empty())
			return false;
		std::map<const char*, size_t>::const_iterator it = idle_index.upper_bound(static_cast<const char*>(p));
		if (it == idle_index.begin())
			return false;
		--it;
		return static_cast<const char*>(p) < it->first + it->second;
	}
	void trim() {
		forbid_while_capturing("returning device memory to the driver");
		for (std::map<size_t, std::vector<void*>>::iterator it = idle.begin(); it != idle.end(); ++it) {
			for (void* p : it->second)
				(void) hipFree(p);
			it->second.clear();
		}
		idle_index.clear();
		idle_bytes = 0;
	}
};
DevicePool g_pool;

/* Device twin of a Parameters object (core/Parameters.hpp:15-95): values plus accumulated gradient.
 * `derived` holds kernel-friendly re-layouts of the values, rebuilt when `version` moves on. */
struct Param {
	size_t rows, cols;
	bool optimizable;
	size_t esize;
	DevBuf values, grad;
	uint64_t version = 1;
	DevBuf derived[3];
	uint64_t derived_version[3] = { 0, 0, 0 };
	int dgrad_layout = 0;              /* which layout derived[1] holds (dgrad_weight_layout) */
	/* A weight matrix: the partial sums of the last weight-gradient launch that was cut into slices (its own and, behind
	 * them, those of the bias gradient). They are added to the gradients when a gradient is first needed - by the
	 * optimizer step as a rule, in one launch for all layers - and until then `pending` lists them (see Deferred). */
	DevBuf partials;
	bool pending = false;
	DevBuf moments[3];                 /* the optimizer's state matrices, allocated (zeroed) on first use */
	int moments_ready = 0;             /* how many of them are */
	double reg_l1 = 0, reg_l2 = 0;     /* ParameterRegularization of the parameter: L1 and L2 lambdas (both 0: none) */
	/* the constraints of StandardParameters (:63-64): clip, max "L1" norm, max "L2" norm of the values and of the gradient; 0 = off */
	double value_limits[3] = { 0, 0, 0 }, grad_limits[3] = { 0, 0, 0 };
	bool constrains_values() const {
		return value_limits[0] > 0 || value_limits[1] > 0 || value_limits[2] > 0;
	}
	bool constrains_grad() const {
		return grad_limits[0] > 0 || grad_limits[1] > 0 || grad_limits[2] > 0;
	}
	~Param();
	Param(size_t rows, size_t cols, bool optimizable, size_t esize) : rows(rows), cols(cols), optimizable(optimizable), esize(esize) {
		values.ensure(bytes());
		grad.ensure(bytes());
		fill_zero(values.p, bytes());
		fill_zero(grad.p, bytes());
	}
	size_t bytes() const {
		return rows * cols * esize;
	}
	std::shared_ptr<Param> deep_copy() const {
		std::shared_ptr<Param> c = std::make_shared<Param>(rows, cols, optimizable, esize);
		copy_in(c->values.p, values.p, CATTLE_HIP_DEVICE, bytes());
		copy_in(c->grad.p, grad.p, CATTLE_HIP_DEVICE, bytes());
		c->reg_l1 = reg_l1;
		c->reg_l2 = reg_l2;
		std::memcpy(c->value_limits, value_limits, sizeof(value_limits));
		std::memcpy(c->grad_limits, grad_limits, sizeof(grad_limits));
		return c;
	}
};

typedef std::shared_ptr<Param> ParamPtr;

/* Sums of weight-gradient slices that have not been added to their gradients yet. Nothing reads a gradient between the
 * backward pass of its layer and the optimizer step (FeedforwardNeuralNetwork.hpp:129-141 runs the layers back to front,
 * SGDOptimizer.hpp:64 is the first reader), so the sums of all layers are taken there in one launch instead of one
 * launch per layer inside the chain of backward launches. Whatever else touches a gradient (reading it, resetting it,
 * its constraints, a deep copy, the next backward pass that would overwrite the partial sums, the start and the end
 * of a recording) settles the sums first. The order of each sum is fixed by reduce_partials_many, so results do not
 * depend on when it is taken. */
struct Deferred {
	struct Entry { Param* owner; ReduceEntry<float> f; ReduceEntry<double> d; };
	std::vector<Entry> entries;
	template<typename T> void add(Param* owner, const ReduceBatch<T>& batch) {
		for (int i = 0; i < batch.count; ++i) {
			Entry e = { owner, {}, {} };
			pick<T>(e) = batch.e[i];
			entries.push_back(e);
		}
		if (batch.count > 0)
			owner->pending = true;
	}
	template<typename T> static ReduceEntry<T>& pick(Entry& e);
	void settle() {
		if (entries.empty())
			return;
		ReduceBatch<float> bf;
		ReduceBatch<double> bd;
		bf.count = bd.count = 0;
		for (Entry& e : entries) {
			e.owner->pending = false;
			if (e.owner->esize == sizeof(float)) {
				bf.e[bf.count++] = e.f;
				if (bf.count == REDUCE_BATCH) {
					reduce_partials_many<float>(bf);
					bf.count = 0;
				}
			} else {
				bd.e[bd.count++] = e.d;
				if (bd.count == REDUCE_BATCH) {
					reduce_partials_many<double>(bd);
					bd.count = 0;
				}
			}
		}
		entries.clear();
		reduce_partials_many<float>(bf);
		reduce_partials_many<double>(bd);
	}
	/* The one entry that waits to be added to `grad`, if it is few enough slices for the optimizer launch to add them on
	 * its way (in the order reduce_partials_many would: for up to as many slices as it has groups of threads that is
	 * plain ascending order); the entry is then taken off the list. Null: none, several, or too many slices. */
	template<typename T> bool take_for_optimizer(const T* grad, ReduceEntry<T>& out) {
		int found = -1;
		for (size_t i = 0; i < entries.size(); ++i)
			if (pick<T>(entries[i]).dst == grad && entries[i].owner->esize == sizeof(T)) {
				if (found >= 0)
					return false;
				found = (int) i;
			}
		if (found < 0)
			return false;
		const ReduceEntry<T>& e = pick<T>(entries[found]);
		const int groups = e.vec ? 16 : 4;          /* reduce_partials_block's GR for 16-byte and for scalar loads */
		if (e.wide || e.splits > std::min(OPT_MAX_PARTS, groups))
			return false;
		out = e;
		Param* owner = entries[found].owner;
		entries.erase(entries.begin() + found);
		bool more = false;
		for (const Entry& o : entries)
			more = more || o.owner == owner;
		owner->pending = more;
		return true;
	}
	/* the owner goes away, and its gradient and partial sums with it */
	void forget(Param* owner) {
		size_t kept = 0;
		for (size_t i = 0; i < entries.size(); ++i)
			if (entries[i].owner != owner)
				entries[kept++] = entries[i];
		entries.resize(kept);
	}
};
template<> ReduceEntry<float>& Deferred::pick<float>(Entry& e) { return e.f; }
template<> ReduceEntry<double>& Deferred::pick<double>(Entry& e) { return e.d; }
Deferred g_deferred;

Param::~Param() {
	if (pending)
		g_deferred.forget(this);
}

template<typename T>
void fill_constant(Param& p, T v) {
	std::vector<T> host(p.rows * p.cols, v);
	copy_in(p.values.p, host.data(), CATTLE_HIP_HOST, p.bytes());
	++p.version;
}

/* enforce_clip_constraint, enforce_l1_norm_constraint, enforce_l2_norm_constraint on the values (set_values,
 * StandardParameters.hpp:105-112) or on the gradient (accumulate_grad, :114-123) */
void constrain(Param& p, bool values) {
	const double* lim = values ? p.value_limits : p.grad_limits;
	void* m = values ? p.values.p : p.grad.p;
	if (p.esize == sizeof(float))
		constrain_matrix<float>(p.rows * p.cols, static_cast<float*>(m), lim[0], lim[1], lim[2]);
	else
		constrain_matrix<double>(p.rows * p.cols, static_cast<double*>(m), lim[0], lim[1], lim[2]);
}

struct LayerBase {
	int dtype;
	size_t in_dims[3], out_dims[3];
	bool input_layer = false;
	bool always_backprop = false;      /* PReLU ignores the input-layer flag */
	std::vector<ParamPtr> params;
	DevBuf in_stage, out_stage, og_stage, ig_stage;
	size_t batch = 0;
	bool have_forward = false;
	uint64_t created;                  /* on the allocation clock: all buffers of the layer are younger */

	LayerBase(int dtype) : dtype(dtype), created(alloc_clock_tick()) { }
	virtual ~LayerBase() { }
	size_t esize() const {
		return dtype == CATTLE_HIP_F32 ? 4 : 8;
	}
	size_t in_volume() const {
		return in_dims[0] * in_dims[1] * in_dims[2];
	}
	size_t out_volume() const {
		return out_dims[0] * out_dims[1] * out_dims[2];
	}
	void copy_base(const LayerBase& o, bool share) {
		std::memcpy(in_dims, o.in_dims, sizeof(in_dims));
		std::memcpy(out_dims, o.out_dims, sizeof(out_dims));
		input_layer = o.input_layer;
		always_backprop = o.always_backprop;
		params.clear();
		for (const ParamPtr& p : o.params)
			params.push_back(share ? p : p->deep_copy());
	}
	virtual LayerBase* clone(bool share) const = 0;
	/* in/out are device pointers; `out` persists until the next forward when it is a stage buffer
	 * or for as long as the caller keeps it (borrowed) */
	virtual void forward(const void* in, size_t N, bool training, void* out) = 0;
	virtual void backward(const void* out_grad, size_t N, void* in_grad) = 0;
	virtual void empty_cache() {
		have_forward = false;
	}
	/* A device tensor that the layer borrowed in its forward pass must still be the caller's in the backward pass: one
	 * that went back to the pool through cattle_hip_free may hold another tensor by now. */
	virtual void check_borrowed() const { }
	static void require_not_released(const void* p) {
		if (g_pool.released(p))
			throw Error(ERR_STATE, "a device tensor that the layer borrowed in its forward pass was freed before the backward pass");
	}
};

int checked_int(size_t v, const char* what) {
	CATTLE_HIP_REQUIRE(v <= 2147483647u, std::string(what) + " exceeds 2^31-1");
	return (int) v;
}

/* ConvKernelLayer and DenseKernelLayer (a dense layer is the 1x1 case on a 1x1 image whose
 * channels are the input volume: X = Map(in.data(), N, volume), DenseKernelLayer.hpp:98). */
template<typename T>
struct ConvLayer : LayerBase {
	ConvShape shape;
	const T* x_cache = nullptr;

	ConvLayer(int dtype, const ConvShape& s, bool dense) : LayerBase(dtype), shape(s) {
		if (dense) {
			in_dims[0] = (size_t) s.C; in_dims[1] = 1; in_dims[2] = 1;
			out_dims[0] = (size_t) s.F; out_dims[1] = 1; out_dims[2] = 1;
		} else {
			in_dims[0] = (size_t) s.H; in_dims[1] = (size_t) s.W; in_dims[2] = (size_t) s.C;
			out_dims[0] = (size_t) s.OH(); out_dims[1] = (size_t) s.OW(); out_dims[2] = (size_t) s.F;
		}
		params.push_back(std::make_shared<Param>((size_t) s.K(), (size_t) s.F, true, sizeof(T)));
		params.push_back(std::make_shared<Param>(1, (size_t) s.F, true, sizeof(T)));
	}
	ConvLayer(const ConvLayer& o, bool share) : LayerBase(o.dtype), shape(o.shape) {
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new ConvLayer(*this, share);
	}
	void forward(const void* in, size_t N, bool, void* out) override {
		const int n = checked_int(N, "batch size");
		const ConvWorkspace ws = conv_workspace<T>(shape, n);
		Param& w = *params[0];
		T* wt = (T*) w.derived[0].ensure(ws.wt_fwd * sizeof(T));
		const bool ready = w.derived_version[0] == w.version;
		conv_forward<T>(shape, n, (const T*) in, (const T*) w.values.p, (const T*) params[1]->values.p, (T*) out, wt, ready);
		w.derived_version[0] = w.version;
		x_cache = (const T*) in;       /* the reference caches the patch matrix (ConvKernelLayer.hpp:127); the input suffices */
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		backward_through(out_grad, N, in_grad, nullptr);
	}
	/* `act`: out_grad is the gradient behind an element-wise activation whose derivative the weight-gradient launch
	 * applies on its way (WgradAct) */
	void backward_through(const void* out_grad, size_t N, void* in_grad, const WgradAct<T>* act) {
		CATTLE_HIP_REQUIRE(x_cache != nullptr, "pass_back without a cached forward input");
		const int n = checked_int(N, "batch size");
		const ConvWorkspace ws = conv_workspace<T>(shape, n);
		Param& w = *params[0];
		T* wt = (T*) w.derived[1].ensure(ws.wt_dgrad * sizeof(T));
		const int layout = dgrad_weight_layout(shape, n);
		const bool ready = w.derived_version[1] == w.version && w.dgrad_layout == layout;
		/* the partial sums of the launch before, if they still wait, would be overwritten */
		if (w.pending)
			g_deferred.settle();
		T* part = (T*) w.partials.ensure(ws.partials * sizeof(T));
		ReduceBatch<T> later;
		conv_backward<T>(shape, n, x_cache, (const T*) w.values.p, (const T*) out_grad, (T*) w.grad.p, (T*) params[1]->grad.p,
				(T*) in_grad, wt, ready, part, act, &later);
		g_deferred.add<T>(&w, later);
		if (in_grad) {
			w.derived_version[1] = w.version;
			w.dgrad_layout = layout;
		}
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		x_cache = nullptr;
	}
	void check_borrowed() const override {
		require_not_released(x_cache);
	}
};

/* TransConvKernelLayer (layer/kernel/TransConvKernelLayer.hpp:143-216). Its forward pass scatters
 * in * W into the output, which is the input gradient of the convolution that maps the output back
 * to the input (same receptor, padding, stride, dilation; channels and filters exchanged) with
 * weights W^T; its backward pass is that convolution's forward pass (input gradient) and weight
 * gradient (transposed). So the three GEMM kernels are reused as they are:
 *   weights W [C x RH*RW*F], column rh + RH*(rw + RW*f)   ->   Wc = W^T, the convolution's [K x C]
 *   bias    [1 x OH*OW*F], one entry per output activation (:52-56). */
template<typename T>
struct TransConvLayer : LayerBase {
	ConvShape conv;                   /* the equivalent convolution: output dims -> input dims */
	const T* x_cache = nullptr;
	DevBuf partials, wgrad_t;

	TransConvLayer(int dtype, const ConvShape& c) : LayerBase(dtype), conv(c) {
		in_dims[0] = (size_t) c.OH(); in_dims[1] = (size_t) c.OW(); in_dims[2] = (size_t) c.F;
		out_dims[0] = (size_t) c.H; out_dims[1] = (size_t) c.W; out_dims[2] = (size_t) c.C;
		params.push_back(std::make_shared<Param>((size_t) c.F, (size_t) c.K(), true, sizeof(T)));
		params.push_back(std::make_shared<Param>(1, out_volume(), true, sizeof(T)));
	}
	TransConvLayer(const TransConvLayer& o, bool share) : LayerBase(o.dtype), conv(o.conv) {
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new TransConvLayer(*this, share);
	}
	/* Wc = W^T, rebuilt when the weights change */
	const T* conv_weights() {
		Param& w = *params[0];
		T* wc = (T*) w.derived[2].ensure(w.bytes());
		if (w.derived_version[2] != w.version) {
			transpose_matrix<T>((int) w.rows, (int) w.cols, (const T*) w.values.p, wc, false);
			w.derived_version[2] = w.version;
		}
		return wc;
	}
	void forward(const void* in, size_t N, bool, void* out) override {
		const int n = checked_int(N, "batch size");
		const ConvWorkspace ws = conv_workspace<T>(conv, n);
		Param& w = *params[0];
		const T* wc = conv_weights();
		T* wt = (T*) w.derived[1].ensure(ws.wt_dgrad * sizeof(T));
		const int layout = dgrad_weight_layout(conv, n);
		conv_input_gradient<T>(conv, n, wc, (const T*) in, (T*) out, wt, w.derived_version[1] == w.version && w.dgrad_layout == layout);
		w.derived_version[1] = w.version;
		w.dgrad_layout = layout;
		add_row_vector<T>(n, out_volume(), (const T*) params[1]->values.p, (T*) out);
		x_cache = (const T*) in;       /* in_mat_cache (:147) */
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		CATTLE_HIP_REQUIRE(x_cache != nullptr, "pass_back without a cached forward input");
		const int n = checked_int(N, "batch size");
		const ConvWorkspace ws = conv_workspace<T>(conv, n);
		Param& w = *params[0];
		accumulate_column_sums<T>(n, out_volume(), (const T*) out_grad, (T*) params[1]->grad.p);      /* :184-185 */
		/* in_mat^T * patches(out_grad) (:208) is the transpose of the convolution's weight gradient */
		T* part = (T*) partials.ensure(ws.partials * sizeof(T));
		T* gt = (T*) wgrad_t.ensure(w.bytes());
		fill_zero(gt, w.bytes());
		conv_weight_gradient<T>(conv, n, (const T*) out_grad, x_cache, gt, (T*) nullptr, part);
		transpose_matrix<T>((int) w.cols, (int) w.rows, gt, (T*) w.grad.p, true);
		if (!in_grad)
			return;
		const T* wc = conv_weights();
		T* wt = (T*) w.derived[0].ensure(ws.wt_fwd * sizeof(T));
		conv_forward<T>(conv, n, (const T*) out_grad, wc, (const T*) nullptr, (T*) in_grad, wt, w.derived_version[0] == w.version);
		w.derived_version[0] = w.version;
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		x_cache = nullptr;
	}
	void check_borrowed() const override {
		require_not_released(x_cache);
	}
};

/* A convolutional LSTM on the device: LSTMNeuralNetwork<Scalar,3,false,false>
 * (neural_network/LSTMNeuralNetwork.hpp:236-503, no multiplicative integration, not stateful, not
 * reversed) whose eight kernels are ConvKernelLayers of one receptor geometry that keep the spatial
 * dimensions (stride 1, output dims = state dims as the constructor asserts, :88-101).
 *
 * The four kernels applied to the same tensor are run as ONE convolution with 4*hidden filters
 * (weights [K x 4*hidden] = [forget | write | candidate | read]; channels are the slowest rank, so
 * the four results are consecutive blocks of the output), and the input-side kernels of all time
 * steps as one launch over a batch of N*T (the sequence tensor (N,T,H,W,C) is that batch as it
 * lies in memory). Gate activations, state update and hidden output of a step are one kernel. The
 * backward pass mirrors it: per step one element-wise kernel and one input-gradient launch for the
 * recurrent kernels; the weight gradients of all steps in two launches at the end.
 *
 * params: 0 = input-side weights [9*C x 4*hidden], 1 = input-side bias [1 x 4*hidden],
 *         2 = output-side (recurrent) weights [9*hidden x 4*hidden], 3 = output-side bias. */
template<typename T>
struct ConvLstm : LayerBase {
	ConvShape sx, sh;               /* input-side and output-side fused convolutions */
	int hidden;
	LstmActs<T> acts;
	bool foremost;
	bool mul_int = false;           /* LSTMNeuralNetwork<Scalar,Rank,MulInt = true> (:44, :303-311) */
	bool fuse_steps = true;         /* run the element-wise part of a step inside the recurrent kernels where the shapes allow */
	int fused_forward_steps = 0, fused_backward_steps = 0;      /* of the last propagate / backpropagate */
	/* alignment of the last propagate (:398-401) */
	size_t T_in = 0, T_out = 0, delay = 0, steps = 0;
	const T* x_cache = nullptr;
	DevBuf zx_all, zh, z, gates, state, act_state, hprev_all, dzx_all, dzh_all, dh, state_grad;
	DevBuf seq_in_stage, seq_out_stage, seq_og_stage, seq_ig_stage;

	ConvLstm(int dtype, const ConvShape& x_shape, const ConvShape& h_shape, const LstmActs<T>& acts, bool foremost) :
			LayerBase(dtype), sx(x_shape), sh(h_shape), hidden(x_shape.F / 4), acts(acts), foremost(foremost) {
		in_dims[0] = (size_t) sx.H; in_dims[1] = (size_t) sx.W; in_dims[2] = (size_t) sx.C;
		out_dims[0] = (size_t) sx.H; out_dims[1] = (size_t) sx.W; out_dims[2] = (size_t) hidden;
		input_layer = foremost;
		params.push_back(std::make_shared<Param>((size_t) sx.K(), (size_t) sx.F, true, sizeof(T)));
		params.push_back(std::make_shared<Param>(1, (size_t) sx.F, true, sizeof(T)));
		params.push_back(std::make_shared<Param>((size_t) sh.K(), (size_t) sh.F, true, sizeof(T)));
		params.push_back(std::make_shared<Param>(1, (size_t) sh.F, true, sizeof(T)));
	}
	ConvLstm(const ConvLstm& o, bool share) : LayerBase(o.dtype), sx(o.sx), sh(o.sh), hidden(o.hidden), acts(o.acts),
			foremost(o.foremost), mul_int(o.mul_int) {
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new ConvLstm(*this, share);
	}
	void forward(const void*, size_t, bool, void*) override {
		throw Error(ERR_STATE, "a recurrent network takes sequences: use cattle_hip_convlstm_propagate");
	}
	void backward(const void*, size_t, void*) override {
		throw Error(ERR_STATE, "a recurrent network takes sequences: use cattle_hip_convlstm_backpropagate");
	}
	/* the gates' pre-activation values are kept for the backward pass only if an activation's derivative reads them */
	bool keeps_z() const {
		for (int i = 0; i < 5; ++i)
			if (act_needs_x(acts.kind[i]))
				return true;
		return false;
	}
	size_t P(size_t N) const {            /* state elements of one step */
		return N * out_volume();
	}
	T* step(DevBuf& b, size_t t, size_t per_step) {
		return (T*) b.p + t * per_step;
	}
	/* propagate (:236-403): input (N, T_in, H, W, C) -> out (N, T_out, H, W, hidden), both on the device */
	void propagate(const T* input, size_t N, size_t in_len, size_t out_len, size_t out_delay, T* out) {
		const int n = checked_int(N, "batch size");
		const size_t total = std::max(in_len, out_len + out_delay);      /* :245-246 */
		const size_t p = P(N), e = sizeof(T);
		checked_int(N * std::max(in_len, total), "batch size times sequence length");
		T_in = in_len; T_out = out_len; delay = out_delay; steps = total;
		/* all input-side kernels of all time steps: one convolution over a batch of N * T_in */
		Param& wx = *params[0];
		Param& wh = *params[2];
		{
			const ConvWorkspace ws = conv_workspace<T>(sx, (int) (N * in_len));
			T* wt = (T*) wx.derived[0].ensure(ws.wt_fwd * e);
			conv_forward<T>(sx, (int) (N * in_len), input, (const T*) wx.values.p, (const T*) params[1]->values.p,
					(T*) zx_all.ensure(4 * p * in_len * e), wt, wx.derived_version[0] == wx.version);
			wx.derived_version[0] = wx.version;
		}
		CATTLE_HIP_REQUIRE((double) (4 * p) * (double) std::max(total, in_len) <= 2147483647.0, "sequence tensor exceeds 2^31-1 elements");
		if (keeps_z())
			z.ensure(4 * p * total * e);
		gates.ensure(4 * p * total * e);
		state.ensure(p * total * e);
		act_state.ensure(p * total * e);
		/* with multiplicative integration the backward pass needs every step's weighted previous output */
		zh.ensure(4 * p * (mul_int ? total : 1) * e);
		/* slab t of hprev_all is the hidden output of step t - 1 (the first step's kernel zeroes slab 0: no previous
		 * output); every slab is written once per pass. The last step's hidden output goes to `out` only. */
		hprev_all.ensure(p * total * e);
		const ConvWorkspace wsh = conv_workspace<T>(sh, n);
		T* wth = (T*) wh.derived[0].ensure(wsh.wt_fwd * e);
		bool fused_steps = fuse_steps;
		fused_forward_steps = 0;
		T* wth_gates = nullptr;             /* the prepared layout of the kernel that runs the step itself */
		for (size_t t = 0; t < total; ++t) {
			const bool has_in = t < in_len, has_prev = t > 0;
			const bool emits = t >= out_delay && t < out_delay + out_len;      /* :386-393 */
			const LstmForwardStep<T> fs = { acts, n, p, has_in ? (const T*) zx_all.p : nullptr, (int) in_len, (int) t, mul_int,
					has_prev ? step(state, t - 1, p) : nullptr, keeps_z() ? step(z, t, 4 * p) : nullptr, step(gates, t, 4 * p),
					step(state, t, p), step(act_state, t, p), (T*) hprev_all.p, (int) total, (int) (t + 1), emits ? out : nullptr,
					(int) out_len, (int) (t - out_delay) };
			/* the previous hidden output where the previous step left it: slab t of (N, total, H, W, hidden) */
			const T* hprev = (const T*) hprev_all.p + N * t;
			if (has_prev && !mul_int && fused_steps) {
				/* the output-side kernels and the element-wise part of the step in one launch where the problem allows:
				 * the weighted previous output then exists only inside that kernel (with multiplicative integration
				 * the backward pass reads it, so it has to be stored) */
				if (!wth_gates)
					wth_gates = (T*) wh.derived[2].ensure(wsh.wt_fwd * e);
				if (conv_forward_lstm<T>(sh, n, hprev, (int) (N * total), (const T*) wh.values.p, (const T*) params[3]->values.p,
						wth_gates, wh.derived_version[2] == wh.version, fs)) {
					wh.derived_version[2] = wh.version;
					++fused_forward_steps;
					continue;
				}
				fused_steps = false;            /* the answer depends on the shapes only: do not ask again */
			}
			T* zh_t = step(zh, mul_int ? t : 0, 4 * p);
			if (has_prev) {
				conv_forward<T>(sh, n, hprev, (const T*) wh.values.p, (const T*) params[3]->values.p, zh_t,
						wth, wh.derived_version[0] == wh.version, (int) (N * total));
				wh.derived_version[0] = wh.version;
			}
			lstm_gates_forward<T>(fs, has_prev ? (const T*) zh_t : nullptr);
		}
		x_cache = input;
		batch = N;
		have_forward = true;
	}
	/* backpropagate (:404-503): out_grad (N, T_out, H, W, hidden) -> in_grad (N, T_in, H, W, C), null if foremost */
	void backpropagate(const T* out_grad, T* in_grad) {
		CATTLE_HIP_REQUIRE(have_forward && x_cache != nullptr, "backpropagate without a matching propagate");
		const size_t N = batch, p = P(N), e = sizeof(T), total = steps;
		const int n = (int) N;
		Param& wx = *params[0];
		Param& wh = *params[2];
		state_grad.ensure(p * e);                                        /* starts at zero (:422-425): the last step's kernel ignores it */
		dh.ensure(p * e);
		dzx_all.ensure(4 * p * T_in * e);
		dzh_all.ensure(4 * p * total * e);                               /* every slab is written; step 0 writes zeros */
		const ConvWorkspace wsh = conv_workspace<T>(sh, n);
		T* wtd = (T*) wh.derived[1].ensure(wsh.wt_dgrad * e);
		auto backward_step = [&](size_t t) {
			const bool has_in = t < T_in, has_prev = t > 0;
			const bool emitted = t >= delay && t < delay + T_out;
			const bool both = mul_int && has_in && has_prev;
			const LstmBackwardStep<T> bs = { acts, n, p, emitted ? out_grad : nullptr, (int) T_out, (int) (t - delay),
					keeps_z() ? step(z, t, 4 * p) : nullptr, step(gates, t, 4 * p), has_prev ? step(state, t - 1, p) : nullptr,
					step(state, t, p), step(act_state, t, p), (T*) state_grad.p, has_in ? (T*) dzx_all.p : nullptr, (int) T_in, (int) t,
					(T*) dzh_all.p, (int) total, (int) t, both ? (const T*) zx_all.p : nullptr,
					both ? (const T*) step(zh, t, 4 * p) : nullptr };
			return bs;
		};
		fused_backward_steps = 0;
		if (total > 0)
			lstm_gates_backward<T>(backward_step(total - 1), (const T*) nullptr);
		for (size_t t = total; t-- > 1;) {
			/* the four output-side kernels' pass_back, summed (:470-473, :491-494), is one input-gradient launch, and
			 * the element-wise part of step t - 1, which is all that reads its result, runs in the kernel that sums the
			 * parts of that launch's reductions when the launch has such a kernel */
			const bool no_fusion = !fuse_steps;
			const LstmBackwardStep<T> before = backward_step(t - 1);
			const bool done = conv_input_gradient<T>(sh, n, (const T*) wh.values.p, (const T*) dzh_all.p + N * t, (T*) dh.p, wtd,
					wh.derived_version[1] == wh.version, no_fusion ? nullptr : &before, (int) (N * total));
			wh.derived_version[1] = wh.version;
			if (done)
				++fused_backward_steps;
			else
				lstm_gates_backward<T>(before, (const T*) dh.p);
		}
		/* parameter gradients of all steps at once: slab 0 of dzh_all and of hprev_all is zero. Each launch leaves the
		 * sum of its slices to whoever reads the gradients first (Deferred). */
		if (wh.pending || wx.pending)
			g_deferred.settle();
		ReduceBatch<T> later;
		if (total > 1) {
			const ConvWorkspace ws = conv_workspace<T>(sh, (int) (N * total));
			conv_weight_gradient<T>(sh, (int) (N * total), (const T*) hprev_all.p, (const T*) dzh_all.p, (T*) wh.grad.p,
					(T*) params[3]->grad.p, (T*) wh.partials.ensure(ws.partials * e), nullptr, &later);
			g_deferred.add<T>(&wh, later);
		}
		{
			const ConvWorkspace ws = conv_workspace<T>(sx, (int) (N * T_in));
			conv_weight_gradient<T>(sx, (int) (N * T_in), x_cache, (const T*) dzx_all.p, (T*) wx.grad.p, (T*) params[1]->grad.p,
					(T*) wx.partials.ensure(ws.partials * e), nullptr, &later);
			g_deferred.add<T>(&wx, later);
			if (in_grad) {
				T* wt = (T*) wx.derived[1].ensure(ws.wt_dgrad * e);
				conv_input_gradient<T>(sx, (int) (N * T_in), (const T*) wx.values.p, (const T*) dzx_all.p, in_grad, wt,
						wx.derived_version[1] == wx.version);
				wx.derived_version[1] = wx.version;
			}
		}
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		x_cache = nullptr;
	}
	void check_borrowed() const override {
		require_not_released(x_cache);
	}
};

template<typename T>
struct BatchNormLayer : LayerBase {
	bool per_last_rank;
	T decay, eps;
	bool stats_init = false;
	DevBuf std_cache, inv_sd_cache, ws;
	bool cache_valid = false;
	size_t cache_batch = 0;         /* batch size of the training pass that filled std_cache and inv_sd_cache */

	BatchNormLayer(int dtype, size_t H, size_t W, size_t C, bool per_last_rank, T decay, T eps) :
			LayerBase(dtype), per_last_rank(per_last_rank), decay(decay), eps(eps) {
		in_dims[0] = out_dims[0] = H;
		in_dims[1] = out_dims[1] = W;
		in_dims[2] = out_dims[2] = C;
		const size_t g = groups();
		params.push_back(std::make_shared<Param>(1, g, false, sizeof(T)));     /* running means */
		params.push_back(std::make_shared<Param>(1, g, false, sizeof(T)));     /* running inverse sds */
		params.push_back(std::make_shared<Param>(1, g, true, sizeof(T)));      /* gammas, OneParameterInitialization */
		params.push_back(std::make_shared<Param>(1, g, true, sizeof(T)));      /* betas, ZeroParameterInitialization */
		fill_constant<T>(*params[2], (T) 1);
	}
	BatchNormLayer(const BatchNormLayer& o, bool share) : LayerBase(o.dtype), per_last_rank(o.per_last_rank), decay(o.decay),
			eps(o.eps), stats_init(o.stats_init) {
		copy_base(o, share);
	}
	size_t groups() const {
		return per_last_rank ? in_dims[2] : in_volume();
	}
	LayerBase* clone(bool share) const override {
		return new BatchNormLayer(*this, share);
	}
	void forward(const void* in, size_t N, bool training, void* out) override {
		const int g = checked_int(groups(), "statistics groups");
		const size_t L = N * in_volume() / groups();
		CATTLE_HIP_REQUIRE(training || stats_init, "inference before any training pass: running statistics unset");
		T* sc = nullptr;
		T* isd = nullptr;
		if (training) {
			sc = (T*) std_cache.ensure(N * in_volume() * sizeof(T));
			isd = (T*) inv_sd_cache.ensure(groups() * sizeof(T));
		}
		T* w = (T*) ws.ensure(bn_workspace(g, L) * sizeof(T));
		bn_forward<T>(g, L, (const T*) in, (const T*) params[2]->values.p, (const T*) params[3]->values.p,
				(T*) params[0]->values.p, (T*) params[1]->values.p, stats_init, training, decay, eps, (T*) out, sc, isd, w);
		if (training) {
			stats_init = true;
			cache_valid = true;
			cache_batch = N;
			++params[0]->version;
			++params[1]->version;
		}
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		CATTLE_HIP_REQUIRE(cache_valid, "pass_back without a training-mode forward pass");
		/* an inference pass in between leaves the caches of the last training pass in place; they only fit a gradient
		 * of that pass's batch size (assert(std_in_mat_cache.rows() == out_grad rows), BatchNormLayer.hpp:194) */
		if (N != cache_batch)
			throw Error(ERR_STATE, "pass_back with a batch size other than that of the last training-mode forward pass");
		const int g = checked_int(groups(), "statistics groups");
		const size_t L = N * in_volume() / groups();
		T* w = (T*) ws.ensure(bn_workspace(g, L) * sizeof(T));
		bn_backward<T>(g, L, (const T*) out_grad, (const T*) params[2]->values.p, (const T*) std_cache.p,
				(const T*) inv_sd_cache.p, (T*) params[2]->grad.p, (T*) params[3]->grad.p, (T*) in_grad, w);
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		cache_valid = false;
		std_cache.release();
	}
};

template<typename T>
struct ActivationLayer : LayerBase {
	int kind;
	T p;
	const T* x_cache = nullptr;
	const T* y_cache = nullptr;

	ActivationLayer(int dtype, int kind, size_t volume, T p) : LayerBase(dtype), kind(kind), p(p) {
		in_dims[0] = out_dims[0] = volume;
		in_dims[1] = out_dims[1] = 1;
		in_dims[2] = out_dims[2] = 1;
		if (kind == CATTLE_HIP_ACT_PRELU || kind == CATTLE_HIP_ACT_PSWISH) {
			params.push_back(std::make_shared<Param>(1, volume, true, sizeof(T)));   /* ConstantParameterInitialization(p) */
			fill_constant<T>(*params[0], p);
		}
		always_backprop = kind == CATTLE_HIP_ACT_PRELU;
	}
	ActivationLayer(const ActivationLayer& o, bool share) : LayerBase(o.dtype), kind(o.kind), p(o.p) {
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new ActivationLayer(*this, share);
	}
	void forward(const void* in, size_t N, bool, void* out) override {
		const size_t total = N * in_volume();
		const int n = checked_int(N, "batch size"), v = checked_int(in_volume(), "volume");
		switch (kind) {
		case CATTLE_HIP_ACT_SOFTMAX:
			softmax_forward<T>(n, v, p, (const T*) in, (T*) out);
			break;
		case CATTLE_HIP_ACT_PRELU:
			prelu_forward<T>(n, v, (const T*) params[0]->values.p, (const T*) in, (T*) out);
			break;
		case CATTLE_HIP_ACT_PSWISH:
			pswish_forward<T>(n, v, (const T*) params[0]->values.p, (const T*) in, (T*) out);
			break;
		default:
			act_forward<T>(kind, total, p, (const T*) in, (T*) out);
		}
		x_cache = (const T*) in;
		y_cache = (const T*) out;
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		CATTLE_HIP_REQUIRE(x_cache != nullptr, "pass_back without a cached forward pass");
		const size_t total = N * in_volume();
		const int n = checked_int(N, "batch size"), v = checked_int(in_volume(), "volume");
		switch (kind) {
		case CATTLE_HIP_ACT_SOFTMAX:
			if (in_grad)
				softmax_backward<T>(n, v, y_cache, (const T*) out_grad, (T*) in_grad);
			break;
		case CATTLE_HIP_ACT_PRELU:
			prelu_backward<T>(n, v, (const T*) params[0]->values.p, x_cache, (const T*) out_grad, (T*) params[0]->grad.p,
					(T*) in_grad);
			break;
		case CATTLE_HIP_ACT_PSWISH:
			pswish_backward<T>(n, v, (const T*) params[0]->values.p, x_cache, (const T*) out_grad, (T*) params[0]->grad.p,
					(T*) in_grad);
			break;
		default:
			if (in_grad)
				act_backward<T>(kind, total, p, x_cache, y_cache, (const T*) out_grad, (T*) in_grad);
		}
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		x_cache = y_cache = nullptr;
	}
	void check_borrowed() const override {
		require_not_released(x_cache);
		require_not_released(y_cache);
	}
};

template<typename T>
struct PoolLayer : LayerBase {
	int kind;
	PoolShape shape;
	DevBuf inds;
	size_t inds_count = 0;

	PoolLayer(int dtype, int kind, const PoolShape& s) : LayerBase(dtype), kind(kind), shape(s) {
		in_dims[0] = (size_t) s.H; in_dims[1] = (size_t) s.W; in_dims[2] = (size_t) s.C;
		out_dims[0] = (size_t) s.OH(); out_dims[1] = (size_t) s.OW(); out_dims[2] = (size_t) s.C;
	}
	PoolLayer(const PoolLayer& o, bool share) : LayerBase(o.dtype), kind(o.kind), shape(o.shape) {
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new PoolLayer(*this, share);
	}
	void forward(const void* in, size_t N, bool, void* out) override {
		const int n = checked_int(N, "batch size");
		checked_int(N * in_volume(), "tensor size");
		if (kind == CATTLE_HIP_POOL_MAX) {
			inds_count = N * out_volume();
			unsigned* ip = (unsigned*) inds.ensure(inds_count * sizeof(unsigned));
			maxpool_forward<T>(shape, n, (const T*) in, (T*) out, ip);
		} else {
			meanpool_forward<T>(shape, n, (const T*) in, (T*) out);
		}
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		if (!in_grad)
			return;
		const int n = checked_int(N, "batch size");
		if (kind == CATTLE_HIP_POOL_MAX) {
			CATTLE_HIP_REQUIRE(inds_count == N * out_volume(), "pass_back without cached max indices");
			maxpool_backward<T>(shape, n, (const T*) out_grad, (const unsigned*) inds.p, (T*) in_grad);
		} else {
			meanpool_backward<T>(shape, n, (const T*) out_grad, (T*) in_grad);
		}
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		inds_count = 0;
		inds.release();
	}
};

/* A kernel layer and the layers a feed-forward network calls right after it (FeedforwardNeuralNetwork.hpp:112-127:
 * layers[i]->pass_forward one after another; backwards :129-141), run as one: convolution or dense -> [per-channel batch
 * norm] -> [element-wise activation] -> [pool]. The member layers stay what they are (their own parameter objects, the
 * running statistics and the arg-max cache of the batch norm and pool layer); this object only replaces the calls.
 *   MODE_ACT   the activation is the GEMM's epilogue (the pool, if any, runs as its own pass);
 *   MODE_POOL  activation and max pooling are the GEMM's epilogue: the full-size activation tensor is never written;
 *   MODE_BN    the GEMM's epilogue also produces the per-tile moments of its output, and one more pass normalises,
 *              activates and pools; the backward pass recomputes the normalised values from the GEMM output;
 *   MODE_UNFUSED  the member layers' own passes, one after another, for everything else (batch sizes or alignments without
 *              16-byte accesses, windows that overlap or do not fit the tiles, parametric activations, softmax).
 * The mode is chosen per forward pass; results do not depend on it beyond rounding. */
enum { MODE_NONE = 0, MODE_UNFUSED = 1, MODE_ACT = 2, MODE_POOL = 3, MODE_BN = 4 };

template<typename T>
struct FusedLayer : LayerBase {
	ConvLayer<T>* conv = nullptr;
	BatchNormLayer<T>* bn = nullptr;
	ActivationLayer<T>* act = nullptr;
	PoolLayer<T>* pool = nullptr;
	std::vector<LayerBase*> members;        /* in call order */
	bool owns_members = false;              /* a clone owns the clones of its members */
	int mode = MODE_NONE;
	bool pool_in_chain = false;             /* MODE_BN: the pool is part of the chain pass */
	bool pool_mean = false;                 /* MODE_POOL: the pool in the GEMM epilogue was a mean pool */
	bool trained = false;                   /* the last forward pass was a training pass (MODE_BN keeps moments only then) */
	const T* y_cache = nullptr;             /* (coded) output the backward pass derives act' from; may be the caller's buffer */
	DevBuf z_buf, pre_buf, dz_buf, stats_buf, mean_buf, chain_ws;
	std::vector<std::unique_ptr<DevBuf>> mid;       /* MODE_UNFUSED: outputs of all members but the last; gradients likewise */
	DevBuf grad_a, grad_b;

	FusedLayer(int dtype, const std::vector<LayerBase*>& layers, bool owns) : LayerBase(dtype), members(layers), owns_members(owns) {
		CATTLE_HIP_REQUIRE(!layers.empty(), "a fused layer needs a kernel layer");
		size_t at = 0;
		conv = dynamic_cast<ConvLayer<T>*>(layers[at]);
		CATTLE_HIP_REQUIRE(conv != nullptr, "the first member must be a convolutional or dense kernel layer of the same scalar type");
		++at;
		if (at < layers.size() && (bn = dynamic_cast<BatchNormLayer<T>*>(layers[at])))
			++at;
		if (at < layers.size() && (act = dynamic_cast<ActivationLayer<T>*>(layers[at])))
			++at;
		if (at < layers.size() && (pool = dynamic_cast<PoolLayer<T>*>(layers[at])))
			++at;
		CATTLE_HIP_REQUIRE(at == layers.size(), "members must be: kernel layer, then optionally batch norm, activation, pool, in this order");
		for (size_t i = 0; i + 1 < layers.size(); ++i)
			CATTLE_HIP_REQUIRE(layers[i]->out_volume() == layers[i + 1]->in_volume(), "member dimensions do not chain");
		std::memcpy(in_dims, conv->in_dims, sizeof(in_dims));
		std::memcpy(out_dims, layers.back()->out_dims, sizeof(out_dims));
		input_layer = conv->input_layer;
		for (LayerBase* l : layers)
			for (const ParamPtr& q : l->params)
				params.push_back(q);
	}
	~FusedLayer() override {
		if (owns_members)
			for (LayerBase* l : members)
				delete l;
	}
	LayerBase* clone(bool share) const override {
		std::vector<LayerBase*> copies;
		for (LayerBase* l : members)
			copies.push_back(l->clone(share));
		FusedLayer* f = new FusedLayer(dtype, copies, true);
		f->input_layer = input_layer;
		return f;
	}

	int OH() const { return conv->shape.OH(); }
	int OW() const { return conv->shape.OW(); }
	int F() const { return conv->shape.F; }
	bool act_fusable() const {
		return !act || act->kind <= CATTLE_HIP_ACT_SWISH;
	}
	/* the pool's windows tile the kernel layer's output exactly */
	bool pool_tiles() const {
		if (!pool)
			return false;
		const PoolShape& ps = pool->shape;
		return ps.H == OH() && ps.W == OW() && ps.C == F() && ps.sv == ps.RH && ps.sh == ps.RW && ps.H % ps.RH == 0 && ps.W % ps.RW == 0;
	}
	bool bn_fusable() const {
		return bn && bn->groups() == (size_t) F();
	}
	ChainShape chain_shape(bool with_pool) const {
		ChainShape cs;
		cs.H = OH(); cs.W = OW(); cs.C = F();
		cs.prh = with_pool ? pool->shape.RH : 1;
		cs.prw = with_pool ? pool->shape.RW : 1;
		cs.pool = with_pool ? (pool->kind == CATTLE_HIP_POOL_MAX ? 1 : 2) : 0;
		cs.kind = act ? act->kind : CATTLE_HIP_ACT_IDENTITY;
		cs.p = act ? (double) act->p : 0.0;
		return cs;
	}
	T* prepared_weights(int n, bool& ready) {
		const ConvWorkspace ws = conv_workspace<T>(conv->shape, n);
		Param& w = *conv->params[0];
		ready = w.derived_version[0] == w.version;
		return (T*) w.derived[0].ensure(ws.wt_fwd * sizeof(T));
	}
	void weights_prepared() {
		Param& w = *conv->params[0];
		w.derived_version[0] = w.version;
	}

	void forward(const void* in, size_t N, bool training, void* out) override {
		const int n = checked_int(N, "batch size");
		const size_t zcount = N * conv->out_volume();
		checked_int(zcount, "tensor size");
		mode = MODE_NONE;
		trained = training;
		const T* x = (const T*) in;
		const T* wv = (const T*) conv->params[0]->values.p;
		const T* bv = (const T*) conv->params[1]->values.p;
		const int kind = act ? act->kind : CATTLE_HIP_ACT_IDENTITY;
		const T ap = act ? act->p : (T) 0;
		Epilogue<T> E = { kind, ap, nullptr, nullptr, 1, 1, OH(), OW(), nullptr, {}, 0, 0 };
		if (members.size() == 1 || !act_fusable() || (bn && !bn_fusable())) {
			forward_unfused(in, N, training, out);
			return;
		}
		bool ready;
		T* wt = prepared_weights(n, ready);
		if (bn) {
			if (bn && !training)
				CATTLE_HIP_REQUIRE(bn->stats_init, "inference before any training pass: running statistics unset");
			T* z = (T*) z_buf.ensure(zcount * sizeof(T));
			int mtiles = 0;
			bool ok = true;
			if (training) {
				E.stats = (T*) stats_buf.ensure(conv_stats_rows(conv->shape, n) * F() * 3 * sizeof(T));
				ok = conv_forward_fused<T>(conv->shape, n, x, wv, bv, z, wt, ready, EPI_STATS, E, &mtiles);
				weights_prepared();
			}
			if (!ok) {
				forward_unfused(in, N, training, out);
				return;
			}
			if (!training) {
				conv_forward<T>(conv->shape, n, x, wv, bv, z, wt, ready);
				weights_prepared();
			}
			pool_in_chain = pool_tiles();
			const ChainShape cs = chain_shape(pool_in_chain);
			T* dst = (T*) out;
			if (pool && !pool_in_chain)
				dst = (T*) pre_buf.ensure(zcount * sizeof(T));      /* the pool's input */
			unsigned* ip = nullptr;
			if (pool_in_chain && pool->kind == CATTLE_HIP_POOL_MAX) {
				pool->inds_count = N * pool->out_volume();
				ip = (unsigned*) pool->inds.ensure(pool->inds_count * sizeof(unsigned));
			}
			T* mean_c = (T*) mean_buf.ensure((size_t) F() * sizeof(T));
			T* isd_c = (T*) bn->inv_sd_cache.ensure((size_t) F() * sizeof(T));
			bn_chain_forward<T>(cs, n, mtiles, training, bn->stats_init, z, E.stats, (const T*) bn->params[2]->values.p,
					(const T*) bn->params[3]->values.p, (T*) bn->params[0]->values.p, (T*) bn->params[1]->values.p, bn->decay, bn->eps,
					mean_c, isd_c, dst, ip);
			if (training) {
				bn->stats_init = true;
				bn->cache_valid = false;        /* the member's own backward pass has nothing to work from */
				++bn->params[0]->version;
				++bn->params[1]->version;
			}
			if (pool && !pool_in_chain)
				pool->forward(dst, N, training, out);
			conv->x_cache = x;
			mode = MODE_BN;
			return;
		}
		const bool needs_pre = !act_backward_from_output(kind, (double) ap);
		if (pool && pool_tiles()) {
			const bool mean = pool->kind == CATTLE_HIP_POOL_MEAN;
			const size_t pcount = N * pool->out_volume();
			E.prh = pool->shape.RH;
			E.prw = pool->shape.RW;
			E.OHp = OH() / E.prh;
			E.OWp = OW() / E.prw;
			if (mean) {
				/* every position of a window takes part in the backward pass: what the activation's derivative reads is
				 * kept at full size (nothing for the kinds whose derivative is a constant) */
				E.pool_mean = 1;
				E.keep_input = needs_pre ? 1 : 0;
				const bool constant_slope = kind == CATTLE_HIP_ACT_IDENTITY || kind == CATTLE_HIP_ACT_SCALED;
				E.pre = constant_slope ? nullptr : (T*) z_buf.ensure(zcount * sizeof(T));
			} else {
				E.inds = (unsigned*) pool->inds.ensure(pcount * sizeof(unsigned));
				E.pre = needs_pre ? (T*) pre_buf.ensure(pcount * sizeof(T)) : nullptr;
			}
			const bool ok = conv_forward_fused<T>(conv->shape, n, x, wv, bv, (T*) out, wt, ready, EPI_POOL, E, nullptr);
			weights_prepared();
			ready = true;
			if (ok) {
				if (!mean)
					pool->inds_count = pcount;
				conv->x_cache = x;
				y_cache = mean ? (const T*) E.pre : (const T*) out;
				pool_mean = mean;
				mode = MODE_POOL;
				return;
			}
			E.inds = nullptr;
			E.pre = nullptr;
			E.pool_mean = E.keep_input = 0;
			E.prh = E.prw = 1;
			E.OHp = OH();
			E.OWp = OW();
		}
		if (act) {
			T* y = pool ? (T*) z_buf.ensure(zcount * sizeof(T)) : (T*) out;
			E.pre = needs_pre ? (T*) pre_buf.ensure(zcount * sizeof(T)) : nullptr;
			const bool ok = conv_forward_fused<T>(conv->shape, n, x, wv, bv, y, wt, ready, EPI_ACT, E, nullptr);
			weights_prepared();
			if (ok) {
				if (pool)
					pool->forward(y, N, training, out);
				conv->x_cache = x;
				y_cache = y;
				mode = MODE_ACT;
				return;
			}
		}
		forward_unfused(in, N, training, out);
	}

	void forward_unfused(const void* in, size_t N, bool training, void* out) {
		while (mid.size() + 1 < members.size())
			mid.push_back(std::unique_ptr<DevBuf>(new DevBuf()));
		const void* cur = in;
		for (size_t i = 0; i < members.size(); ++i) {
			LayerBase* l = members[i];
			void* dst = i + 1 == members.size() ? out : mid[i]->ensure(N * l->out_volume() * esize());
			l->forward(cur, N, training, dst);
			cur = dst;
		}
		mode = MODE_UNFUSED;
	}

	void backward(const void* out_grad, size_t N, void* in_grad) override {
		CATTLE_HIP_REQUIRE(mode != MODE_NONE, "pass_back without a cached forward pass");
		const int n = checked_int(N, "batch size");
		const size_t zcount = N * conv->out_volume();
		if (mode == MODE_UNFUSED) {
			const void* g = out_grad;
			for (size_t i = members.size(); i-- > 0;) {
				LayerBase* l = members[i];
				void* dst = in_grad;
				if (i > 0)
					dst = ((members.size() - i) % 2 ? grad_a : grad_b).ensure(N * l->in_volume() * esize());
				l->backward(g, N, dst);
				g = dst;
			}
			return;
		}
		const T* g = (const T*) out_grad;
		T* dz = (T*) dz_buf.ensure(zcount * sizeof(T));
		if (mode == MODE_BN) {
			if (!trained)
				throw Error(ERR_STATE, "pass_back without a training-mode forward pass");
			if (pool && !pool_in_chain) {
				T* gp = (T*) grad_a.ensure(zcount * sizeof(T));
				pool->backward(g, N, gp);
				g = gp;
			}
			const ChainShape cs = chain_shape(pool_in_chain);
			T* ws = (T*) chain_ws.ensure(bn_chain_workspace(F()) * sizeof(T));
			bn_chain_backward<T>(cs, n, g, pool_in_chain ? (const unsigned*) pool->inds.p : nullptr, (const T*) z_buf.p,
					(const T*) bn->params[2]->values.p, (const T*) bn->params[3]->values.p, (const T*) mean_buf.p,
					(const T*) bn->inv_sd_cache.p, (T*) bn->params[2]->grad.p, (T*) bn->params[3]->grad.p, dz, ws);
		} else if (mode == MODE_POOL && pool_mean) {
			/* y_cache is the full-size tensor of what the derivative reads: inputs or coded outputs of the activation */
			chain_backward<T>(chain_shape(true), n, g, nullptr, needs_pre() ? nullptr : y_cache, needs_pre() ? y_cache : nullptr, dz);
		} else if (mode == MODE_POOL) {
			CATTLE_HIP_REQUIRE(pool->inds_count == N * pool->out_volume(), "pass_back without cached max indices");
			if (pooled_weight_gradient(g, n, in_grad))
				return;
			chain_backward<T>(chain_shape(true), n, g, (const unsigned*) pool->inds.p, y_cache, needs_pre() ? (const T*) pre_buf.p : nullptr, dz);
		} else {
			if (pool) {
				T* gp = (T*) grad_a.ensure(zcount * sizeof(T));
				pool->backward(g, N, gp);
				g = gp;
			}
			if (act && act_sign_coded(act->kind) && act->p >= 0) {
				/* a rectifier, whose derivative the sign bit of the coded output names: applied by the weight-gradient
				 * launch while it loads the gradient, which also leaves dz behind for the input-gradient launch - no
				 * pass of its own */
				const WgradAct<T> through = { y_cache, in_grad ? dz : nullptr, act->kind, (T) act->p, nullptr, 0, 0 };
				conv->backward_through(g, N, in_grad, &through);
				return;
			}
			chain_backward<T>(chain_shape(false), n, g, nullptr, y_cache, needs_pre() ? (const T*) pre_buf.p : nullptr, dz);
		}
		conv->backward(dz, N, in_grad);
	}
	bool needs_pre() const {
		return act && !act_backward_from_output(act->kind, (double) act->p);
	}
	/* MODE_POOL with max pooling, nobody needing the input gradient (a network's first layer), no activation or a
	 * rectifier, windows whose sides are powers of two, 16-byte loads: the weight-gradient launch forms the gradient
	 * of the kernel layer's output from the pooled gradient, the arg-max cache and the coded outputs as it loads its
	 * operand, and the pass over the full-size tensor that scatters it (chain_backward_kernel) does not run. */
	bool pooled_weight_gradient(const T* g, int n, void* in_grad) {
		auto log2_exact = [](int v) {
			int s = 0;
			while ((1 << s) < v)
				++s;
			return (1 << s) == v ? s : -1;
		};
		const PoolShape& ps = pool->shape;
		const int sh_a = log2_exact(ps.RH), sh_b = log2_exact(ps.RW);
		constexpr int V = 16 / (int) sizeof(T);
		auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
		if (in_grad != nullptr || sh_a < 0 || sh_b < 0 || n % V != 0 || !aligned(g) || !aligned(y_cache) || !aligned(pool->inds.p) ||
				!aligned(conv->x_cache))
			return false;
		if (act && !(act_sign_coded(act->kind) && act->p >= 0))
			return false;
		const WgradAct<T> through = { y_cache, nullptr, act ? act->kind : -1, act ? (T) act->p : (T) 0, (const unsigned*) pool->inds.p, sh_a, sh_b };
		conv->backward_through(g, (size_t) n, nullptr, &through);
		return true;
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		for (LayerBase* l : members)
			l->empty_cache();
		mode = MODE_NONE;
		y_cache = nullptr;
		z_buf.release();
		pre_buf.release();
		dz_buf.release();
		grad_a.release();
		grad_b.release();
		mid.clear();
	}
	void check_borrowed() const override {
		if (mode == MODE_UNFUSED) {
			for (LayerBase* l : members)
				l->check_borrowed();
			return;
		}
		require_not_released(conv->x_cache);
		if (y_cache)
			require_not_released(y_cache);
	}
};

/* DropoutLayer (layer/DropoutLayer.hpp:33-96). The mask of a training pass is not kept: the pass number is, and the
 * backward pass regenerates the mask from it. An inference pass hands the input through. */
template<typename T>
struct DropoutLayer : LayerBase {
	T prob, eps;
	unsigned long long seed, passes = 0;      /* training passes so far; the last one's number is passes - 1 */
	bool have_mask = false;

	DropoutLayer(int dtype, size_t volume, T prob, T eps, unsigned long long seed) : LayerBase(dtype), prob(prob), eps(eps),
			seed(seed) {
		in_dims[0] = out_dims[0] = volume;
		in_dims[1] = out_dims[1] = 1;
		in_dims[2] = out_dims[2] = 1;
	}
	DropoutLayer(const DropoutLayer& o, bool share) : LayerBase(o.dtype), prob(o.prob), eps(o.eps), seed(o.seed),
			passes(o.passes), have_mask(o.have_mask) {
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new DropoutLayer(*this, share);
	}
	void forward(const void* in, size_t N, bool training, void* out) override {
		const size_t total = N * in_volume();
		if (training) {
			/* the mask's key, a function of the number of the pass, is an argument of the kernel: a recorded launch
			 * would draw the same mask at every replay */
			forbid_while_capturing("a training pass of a dropout layer (its mask changes from pass to pass; record the layers around it)");
			dropout_apply<T>(total, dropout_pass_key(seed, passes), prob, eps, (const T*) in, (T*) out);
			++passes;
			have_mask = true;
		} else if (in != out)
			CATTLE_HIP_CHECK(hipMemcpyAsync(out, in, total * sizeof(T), hipMemcpyDeviceToDevice, stream()));
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		/* assert(dropout_mask.dimension(0) == out_grad.dimension(0)), DropoutLayer.hpp:91 */
		CATTLE_HIP_REQUIRE(have_mask, "pass_back without a training pass_forward");
		if (in_grad)
			dropout_apply<T>(N * in_volume(), dropout_pass_key(seed, passes - 1), prob, eps, (const T*) out_grad, (T*) in_grad);
	}
	void empty_cache() override {
		LayerBase::empty_cache();
		have_mask = false;
	}
};

/* ReshapeLayer (layer/ReshapeLayer.hpp:31-90): the same values under other dimensions; in column-major memory with
 * the sample index first that is a copy. */
struct ReshapeLayer : LayerBase {
	ReshapeLayer(int dtype, const size_t in[3], const size_t out[3]) : LayerBase(dtype) {
		std::memcpy(in_dims, in, sizeof(in_dims));
		std::memcpy(out_dims, out, sizeof(out_dims));
	}
	ReshapeLayer(const ReshapeLayer& o, bool share) : LayerBase(o.dtype) {
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new ReshapeLayer(*this, share);
	}
	void forward(const void* in, size_t N, bool, void* out) override {
		if (in != out)
			CATTLE_HIP_CHECK(hipMemcpyAsync(out, in, N * in_volume() * esize(), hipMemcpyDeviceToDevice, stream()));
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		if (in_grad && in_grad != out_grad)
			CATTLE_HIP_CHECK(hipMemcpyAsync(in_grad, out_grad, N * in_volume() * esize(), hipMemcpyDeviceToDevice, stream()));
	}
};

/* BroadcastLayer (layer/BroadcastLayer.hpp:31-101) */
template<typename T>
struct BroadcastLayer : LayerBase {
	int reps[3];

	BroadcastLayer(int dtype, const size_t in[3], const size_t broadcast[3]) : LayerBase(dtype) {
		for (int i = 0; i < 3; ++i) {
			in_dims[i] = in[i];
			out_dims[i] = in[i] * broadcast[i];
			reps[i] = (int) broadcast[i];
		}
	}
	BroadcastLayer(const BroadcastLayer& o, bool share) : LayerBase(o.dtype) {
		std::memcpy(reps, o.reps, sizeof(reps));
		copy_base(o, share);
	}
	LayerBase* clone(bool share) const override {
		return new BroadcastLayer(*this, share);
	}
	void forward(const void* in, size_t N, bool, void* out) override {
		broadcast_forward<T>((int) in_dims[0], (int) in_dims[1], (int) in_dims[2], reps[0], reps[1], reps[2],
				checked_int(N, "batch size"), (const T*) in, (T*) out);
	}
	void backward(const void* out_grad, size_t N, void* in_grad) override {
		if (in_grad)
			broadcast_backward<T>((int) in_dims[0], (int) in_dims[1], (int) in_dims[2], reps[0], reps[1], reps[2],
					checked_int(N, "batch size"), (const T*) out_grad, (T*) in_grad);
	}
};

struct Timer {
	hipEvent_t start = nullptr, stop = nullptr;
};

/* A recorded sequence of library calls (kernels and device-to-device copies on the library's stream) that can be
 * launched again as one unit. It keeps the blocks that were given back to the pool while it was recorded. */
struct Graph {
	hipGraph_t graph = nullptr;
	hipGraphExec_t exec = nullptr;
	std::vector<void*> blocks;
	uint64_t recorded_at = 0;          /* on the allocation clock: older allocations are pinned while the graph lives */
};

LayerBase* as_layer(cattle_hip_layer_t h) {
	CATTLE_HIP_REQUIRE(h != nullptr, "null layer handle");
	return reinterpret_cast<LayerBase*>(h);
}

Param& param_at(LayerBase* l, size_t index) {
	CATTLE_HIP_REQUIRE(index < l->params.size(), "parameter index out of range");
	return *l->params[index];
}

void check_dtype(int dtype) {
	CATTLE_HIP_REQUIRE(dtype == CATTLE_HIP_F32 || dtype == CATTLE_HIP_F64, "dtype must be CATTLE_HIP_F32 or CATTLE_HIP_F64");
}

void check_space(int space) {
	CATTLE_HIP_REQUIRE(space == CATTLE_HIP_HOST || space == CATTLE_HIP_DEVICE, "memspace must be HOST or DEVICE");
}

template<typename Fn>
int guarded(Fn fn) {
	std::lock_guard<std::recursive_mutex> lock(g_mutex);
	try {
		ensure_init(0);
		fn();
		return CATTLE_HIP_OK;
	} catch (const Error& e) {
		g_last_error = e.what();
		return e.code;
	} catch (const std::bad_alloc&) {
		g_last_error = "host allocation failed";
		return CATTLE_HIP_ERR_OOM;
	} catch (const std::exception& e) {
		g_last_error = e.what();
		return CATTLE_HIP_ERR_INVALID;
	}
}

/* Staging for the loss entry points when the caller's buffers are host memory. */
struct LossStage {
	DevBuf out, obj, dst;
};
LossStage g_loss_stage;

template<typename T>
void run_loss(bool grad_pass, int kind, const void* out, int out_space, const void* obj, int obj_space, size_t batch,
		size_t time_steps, size_t sample_size, double epsilon, double scale, void* dst, int dst_space) {
	const size_t limit = 2147483647u;
	CATTLE_HIP_REQUIRE(batch <= limit && time_steps <= limit / batch && sample_size <= limit / (batch * time_steps),
			"tensor exceeds 2^31-1 elements");
	const size_t count = batch * time_steps * sample_size;
	const size_t bytes = count * sizeof(T), dst_bytes = grad_pass ? bytes : batch * sizeof(T);
	const T* out_dev = static_cast<const T*>(out);
	const T* obj_dev = static_cast<const T*>(obj);
	if (out_space == CATTLE_HIP_HOST) {
		copy_in(g_loss_stage.out.ensure(bytes), out, CATTLE_HIP_HOST, bytes);
		out_dev = static_cast<const T*>(g_loss_stage.out.p);
	}
	if (obj_space == CATTLE_HIP_HOST) {
		copy_in(g_loss_stage.obj.ensure(bytes), obj, CATTLE_HIP_HOST, bytes);
		obj_dev = static_cast<const T*>(g_loss_stage.obj.p);
	}
	T* dst_dev = dst_space == CATTLE_HIP_HOST ? static_cast<T*>(g_loss_stage.dst.ensure(dst_bytes)) : static_cast<T*>(dst);
	if (grad_pass)
		loss_d_function<T>(kind, (int) batch, (int) time_steps, (int) sample_size, (T) epsilon, (T) scale, out_dev, obj_dev,
				dst_dev);
	else
		loss_function<T>(kind, (int) batch, (int) time_steps, (int) sample_size, (T) epsilon, out_dev, obj_dev, dst_dev);
	if (dst_space == CATTLE_HIP_HOST)
		copy_out(dst, CATTLE_HIP_HOST, dst_dev, dst_bytes);
}

void loss_entry(bool grad_pass, int dtype, int kind, const void* out, int out_space, const void* obj, int obj_space,
		size_t batch, size_t time_steps, size_t sample_size, double epsilon, double scale, void* dst, int dst_space) {
	check_dtype(dtype);
	check_space(out_space);
	check_space(obj_space);
	check_space(dst_space);
	CATTLE_HIP_REQUIRE((kind & ~CATTLE_HIP_LOSS_NEGATED) >= 0 && (kind & ~CATTLE_HIP_LOSS_NEGATED) < LOSS_KINDS, "unknown loss kind");
	CATTLE_HIP_REQUIRE((kind & ~CATTLE_HIP_LOSS_NEGATED) != CATTLE_HIP_LOSS_BINARY_CROSS_ENTROPY || sample_size == 1,
			"the binary cross entropy loss takes one value per sample and time step");
	CATTLE_HIP_REQUIRE(out != nullptr && obj != nullptr && dst != nullptr, "null tensor buffer");
	CATTLE_HIP_REQUIRE(batch > 0 && time_steps > 0 && sample_size > 0, "batch, time steps and sample size must be positive");
	if (dtype == CATTLE_HIP_F32)
		run_loss<float>(grad_pass, kind, out, out_space, obj, obj_space, batch, time_steps, sample_size, epsilon, scale, dst,
				dst_space);
	else
		run_loss<double>(grad_pass, kind, out, out_space, obj, obj_space, batch, time_steps, sample_size, epsilon, scale, dst,
				dst_space);
}

Param& optimizable_param(cattle_hip_layer_t layer, size_t index) {
	Param& p = param_at(as_layer(layer), index);
	CATTLE_HIP_REQUIRE(p.optimizable, "the parameters are not optimizable");
	return p;
}

/* One optimizer update of a parameter, optionally followed (in the same kernel) by the reset of its gradient. */
void run_optimizer(cattle_hip_layer_t layer, size_t index, cattle_hip_optimizer optimizer, const double hyper[4], size_t epoch,
		size_t timestep, bool reset_grad) {
	Param& p = optimizable_param(layer, index);
	CATTLE_HIP_REQUIRE(hyper != nullptr, "null hyper-parameter array");
	g_deferred.settle();
	const int states = optimizer_state_count((int) optimizer);
	for (int i = p.moments_ready; i < states; ++i) {
		fill_zero(p.moments[i].ensure(p.bytes()), p.bytes());
		p.moments_ready = i + 1;
	}
	const size_t n = p.rows * p.cols;
	/* the step form is SGDOptimizer::_train's regularize + update + reset; the plain update is _update_params alone */
	double l1 = reset_grad ? p.reg_l1 : 0, l2 = reset_grad ? p.reg_l2 : 0;
	if (p.constrains_grad() && (l1 != 0 || l2 != 0)) {
		/* Parameters::regularize is an accumulate_grad: the constraints apply to gradient + regularization */
		if (p.esize == sizeof(float))
			add_regularization<float>(n, static_cast<const float*>(p.values.p), static_cast<float*>(p.grad.p), (float) l1, (float) l2);
		else
			add_regularization<double>(n, static_cast<const double*>(p.values.p), static_cast<double*>(p.grad.p), l1, l2);
		constrain(p, false);
		l1 = l2 = 0;
	}
	if (p.esize == sizeof(float))
		optimizer_update<float>((int) optimizer, hyper, epoch, timestep, n, static_cast<float*>(p.grad.p),
				static_cast<float*>(p.moments[0].p), static_cast<float*>(p.moments[1].p), static_cast<float*>(p.moments[2].p),
				static_cast<float*>(p.values.p), reset_grad, (float) l1, (float) l2);
	else
		optimizer_update<double>((int) optimizer, hyper, epoch, timestep, n, static_cast<double*>(p.grad.p),
				static_cast<double*>(p.moments[0].p), static_cast<double*>(p.moments[1].p),
				static_cast<double*>(p.moments[2].p), static_cast<double*>(p.values.p), reset_grad, l1, l2);
	if (p.constrains_values())
		constrain(p, true);              /* the optimizers hand the new values to set_values */
	++p.version;
}

/* The update + gradient reset of many parameters, OPT_BATCH per launch. A parameter shared by several of the listed
 * layers is updated once. Weight matrices of convolution and dense layers whose prepared layouts are current have
 * them rewritten by the same kernel and stay current. */
template<typename T>
void run_optimizer_many(const cattle_hip_layer_t* layers, const size_t* indices, size_t count, cattle_hip_optimizer optimizer,
		const double hyper[4], size_t epoch, size_t timestep) {
	const int states = optimizer_state_count((int) optimizer);
	/* The gradients become whole here. Partial sums of few slices ride along with the update of their parameter; the
	 * others are added to their gradients first, in one launch for all layers. */
	std::vector<Param*> seen, limited;
	std::vector<std::pair<Param*, ReduceEntry<T>>> riding;
	for (size_t i = 0; i < count; ++i) {
		Param& p = optimizable_param(layers[i], indices[i]);
		ReduceEntry<T> e;
		if (p.esize == sizeof(T) && !p.constrains_grad() && g_deferred.take_for_optimizer<T>(static_cast<const T*>(p.grad.p), e))
			riding.push_back(std::make_pair(&p, e));
	}
	g_deferred.settle();
	OptBatch<T> batch;
	batch.count = 0;
	auto flush = [&] {
		optimizer_step_many<T>((int) optimizer, hyper, epoch, timestep, batch);
		batch.count = 0;
	};
	for (size_t i = 0; i < count; ++i) {
		Param& p = optimizable_param(layers[i], indices[i]);
		CATTLE_HIP_REQUIRE(p.esize == sizeof(T), "parameters of one optimizer step must share a scalar type");
		if (std::find(seen.begin(), seen.end(), &p) != seen.end())
			continue;
		seen.push_back(&p);
		for (int m = p.moments_ready; m < states; ++m) {
			fill_zero(p.moments[m].ensure(p.bytes()), p.bytes());
			p.moments_ready = m + 1;
		}
		OptParam<T>& q = batch.p[batch.count++];
		q.grad = static_cast<T*>(p.grad.p);
		q.values = static_cast<T*>(p.values.p);
		q.s0 = static_cast<T*>(p.moments[0].p);
		q.s1 = static_cast<T*>(p.moments[1].p);
		q.s2 = static_cast<T*>(p.moments[2].p);
		q.n = p.rows * p.cols;
		q.l1 = (T) p.reg_l1;
		q.l2 = (T) p.reg_l2;
		q.parts = nullptr;
		q.splits = 0;
		for (const std::pair<Param*, ReduceEntry<T>>& r : riding)
			if (r.first == &p) {
				q.parts = r.second.partials;
				q.splits = r.second.splits;
			}
		if (p.constrains_grad() && (p.reg_l1 != 0 || p.reg_l2 != 0)) {
			add_regularization<T>(p.rows * p.cols, static_cast<const T*>(p.values.p), static_cast<T*>(p.grad.p), q.l1, q.l2);
			constrain(p, false);
			q.l1 = q.l2 = (T) 0;
		}
		q.wt_fwd = q.wt_dgrad = nullptr;
		q.K = q.RHW = 1;
		q.ldw_fwd = q.ldw_dgrad = 0;
		const ConvLayer<T>* conv = dynamic_cast<const ConvLayer<T>*>(as_layer(layers[i]));
		bool fwd_current = false, dgrad_current = false;
		if (p.constrains_values()) {
			limited.push_back(&p);         /* constrained after the update; the prepared layouts are rebuilt from the result */
		} else if (conv && indices[i] == 0) {
			const ConvShape& cs = conv->shape;
			fwd_current = p.derived[0].p && p.derived_version[0] == p.version;
			dgrad_current = p.derived[1].p && p.derived_version[1] == p.version && p.dgrad_layout == 0;
			q.K = cs.K();
			q.RHW = cs.RH * cs.RW;
			q.ldw_fwd = prepared_weight_row_length(cs.F);
			q.ldw_dgrad = prepared_weight_row_length(cs.C);
			if (fwd_current)
				q.wt_fwd = static_cast<T*>(p.derived[0].p);
			if (dgrad_current)
				q.wt_dgrad = static_cast<T*>(p.derived[1].p);
		}
		++p.version;
		if (fwd_current)
			p.derived_version[0] = p.version;
		if (dgrad_current)
			p.derived_version[1] = p.version;
		if (batch.count == OPT_BATCH)
			flush();
	}
	flush();
	for (Param* p : limited)
		constrain(*p, true);
}



template<typename T>
void convlstm_propagate(ConvLstm<T>* l, const void* input, int in_space, size_t batch, size_t in_len, size_t out_len,
		size_t delay, void* out, int out_space) {
	const size_t in_bytes = batch * in_len * l->in_volume() * sizeof(T), out_bytes = batch * out_len * l->out_volume() * sizeof(T);
	const void* in_dev = input;
	if (in_space == CATTLE_HIP_HOST) {
		copy_in(l->seq_in_stage.ensure(in_bytes), input, CATTLE_HIP_HOST, in_bytes);
		in_dev = l->seq_in_stage.p;
	}
	void* out_dev = out_space == CATTLE_HIP_HOST ? l->seq_out_stage.ensure(out_bytes) : out;
	l->have_forward = false;
	l->propagate((const T*) in_dev, batch, in_len, out_len, delay, (T*) out_dev);
	if (out_space == CATTLE_HIP_HOST)
		copy_out(out, CATTLE_HIP_HOST, out_dev, out_bytes);
}

template<typename T>
void convlstm_backpropagate(ConvLstm<T>* l, const void* out_grad, int og_space, void* in_grad, int ig_space) {
	if (!l->have_forward)
		throw Error(ERR_STATE, "backpropagate without a matching propagate");
	l->check_borrowed();
	const size_t og_bytes = l->batch * l->T_out * l->out_volume() * sizeof(T), ig_bytes = l->batch * l->T_in * l->in_volume() * sizeof(T);
	const void* og_dev = out_grad;
	if (og_space == CATTLE_HIP_HOST) {
		copy_in(l->seq_og_stage.ensure(og_bytes), out_grad, CATTLE_HIP_HOST, og_bytes);
		og_dev = l->seq_og_stage.p;
	}
	void* ig_dev = nullptr;
	if (in_grad)
		ig_dev = ig_space == CATTLE_HIP_HOST ? l->seq_ig_stage.ensure(ig_bytes) : in_grad;
	l->backpropagate((const T*) og_dev, (T*) ig_dev);
	if (in_grad && ig_space == CATTLE_HIP_HOST)
		copy_out(in_grad, CATTLE_HIP_HOST, ig_dev, ig_bytes);
}

/* kernel index in the order of LSTMNeuralNetwork::populate_layer_vector (:521-529): input_forget, output_forget,
 * input_write, output_write, input_candidate, output_candidate, input_read, output_read; `bias` picks the bias.
 * Returns the fused parameter and the byte range of the kernel's block of columns in it. */
Param& lstm_kernel_param(cattle_hip_layer_t lstm, size_t kernel, int bias, size_t& offset, size_t& bytes) {
	LayerBase* l = as_layer(lstm);
	CATTLE_HIP_REQUIRE(dynamic_cast<ConvLstm<float>*>(l) || dynamic_cast<ConvLstm<double>*>(l), "not a ConvLSTM handle");
	CATTLE_HIP_REQUIRE(kernel < 8, "kernel index out of range");
	Param& p = *l->params[(kernel % 2) * 2 + (bias ? 1 : 0)];
	const size_t gate = kernel / 2, block = p.rows * (p.cols / 4);
	offset = gate * block * p.esize;
	bytes = block * p.esize;
	return p;
}


} /* namespace */

hipStream_t stream() {
	return g_stream;
}

uint64_t alloc_clock_tick() {
	return ++g_alloc_clock;
}

bool pinned_by_graph(uint64_t born) {
	return born < newest_live_graph();
}

void park_allocation(void* p, uint64_t born) {
	g_parked.push_back(Parked{ p, born });
}

bool capturing() {
	return g_capturing;
}

void forbid_while_capturing(const char* what) {
	if (g_capturing)
		throw Error(ERR_STATE, std::string("not possible while a graph is being recorded: ") + what);
}

} /* namespace cattle_hip */

using namespace cattle_hip;

extern "C" {

int cattle_hip_init(int device) {
	std::lock_guard<std::recursive_mutex> lock(g_mutex);
	try {
		ensure_init(device);
		return CATTLE_HIP_OK;
	} catch (const Error& e) {
		g_last_error = e.what();
		return e.code;
	}
}

const char* cattle_hip_last_error(void) {
	return g_last_error.c_str();
}

int cattle_hip_synchronize(void) {
	return guarded([&] {
		forbid_while_capturing("waiting for the device");
		CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
	});
}

int cattle_hip_alloc(void** device_ptr, size_t bytes) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(device_ptr != nullptr, "null output pointer");
		*device_ptr = g_pool.take(bytes);
	});
}

int cattle_hip_free(void* device_ptr) {
	return guarded([&] {
		if (device_ptr)
			g_pool.give_back(device_ptr);
	});
}

int cattle_hip_trim(void) {
	return guarded([&] {
		forbid_while_capturing("waiting for the device");
		CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
		g_pool.trim();
	});
}

int cattle_hip_memory_info(size_t* free_bytes, size_t* total_bytes) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(free_bytes != nullptr && total_bytes != nullptr, "null output pointer");
		forbid_while_capturing("waiting for the device");
		CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
		CATTLE_HIP_CHECK(hipMemGetInfo(free_bytes, total_bytes));
	});
}

int cattle_hip_upload(void* dst_device, const void* src_host, size_t bytes) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(bytes == 0 || (dst_device && src_host), "null buffer");
		copy_in(dst_device, src_host, CATTLE_HIP_HOST, bytes);
	});
}

int cattle_hip_download(void* dst_host, const void* src_device, size_t bytes) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(bytes == 0 || (dst_host && src_device), "null buffer");
		copy_out(dst_host, CATTLE_HIP_HOST, src_device, bytes);
	});
}

int cattle_hip_fill_zero(void* dst_device, size_t bytes) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(bytes == 0 || dst_device, "null buffer");
		fill_zero(dst_device, bytes);
	});
}

int cattle_hip_timer_create(cattle_hip_timer_t* timer) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(timer != nullptr, "null output pointer");
		std::unique_ptr<Timer> t(new Timer());
		CATTLE_HIP_CHECK(hipEventCreate(&t->start));
		CATTLE_HIP_CHECK(hipEventCreate(&t->stop));
		*timer = reinterpret_cast<cattle_hip_timer_t>(t.release());
	});
}

int cattle_hip_timer_destroy(cattle_hip_timer_t timer) {
	return guarded([&] {
		Timer* t = reinterpret_cast<Timer*>(timer);
		if (t) {
			(void) hipEventDestroy(t->start);
			(void) hipEventDestroy(t->stop);
			delete t;
		}
	});
}

int cattle_hip_timer_start(cattle_hip_timer_t timer) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(timer != nullptr, "null timer");
		forbid_while_capturing("timing");
		CATTLE_HIP_CHECK(hipEventRecord(reinterpret_cast<Timer*>(timer)->start, stream()));
	});
}

int cattle_hip_timer_stop(cattle_hip_timer_t timer, float* elapsed_ms) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(timer != nullptr && elapsed_ms != nullptr, "null timer or output");
		Timer* t = reinterpret_cast<Timer*>(timer);
		forbid_while_capturing("timing");
		CATTLE_HIP_CHECK(hipEventRecord(t->stop, stream()));
		CATTLE_HIP_CHECK(hipEventSynchronize(t->stop));
		CATTLE_HIP_CHECK(hipEventElapsedTime(elapsed_ms, t->start, t->stop));
	});
}

int cattle_hip_graph_begin_capture(void) {
	return guarded([&] {
		if (g_capturing)
			throw Error(ERR_STATE, "a graph is already being recorded");
		g_deferred.settle();            /* nothing pending crosses into the recording ... */
		CATTLE_HIP_CHECK(hipStreamBeginCapture(stream(), hipStreamCaptureModeRelaxed));
		g_capturing = true;
	});
}

int cattle_hip_graph_end_capture(cattle_hip_graph_t* graph) {
	return guarded([&] {
		if (!g_capturing)
			throw Error(ERR_STATE, "no graph is being recorded");
		/* ... or out of it: what the recorded passes left pending is summed by the recording itself, so that a launch
		 * of the graph leaves whole gradients whatever the host does next */
		bool settled = true;
		try {
			g_deferred.settle();
		} catch (const Error&) {
			settled = false;
		}
		g_capturing = false;
		std::unique_ptr<Graph> gr(new Graph());
		/* blocks freed during the recording stay out of circulation, whatever becomes of the graph */
		gr->blocks.swap(g_pool.held);
		for (void* b : g_pool.taken)
			g_pool.owner[b] = &gr->blocks;
		g_pool.taken.clear();
		hipError_t e = hipStreamEndCapture(stream(), &gr->graph);
		if (e == hipSuccess && !settled)
			e = hipErrorUnknown;
		if (e == hipSuccess && gr->graph != nullptr)
			e = hipGraphInstantiate(&gr->exec, gr->graph, nullptr, nullptr, 0);
		if (e != hipSuccess || gr->graph == nullptr || graph == nullptr) {
			if (gr->exec)
				(void) hipGraphExecDestroy(gr->exec);
			if (gr->graph)
				(void) hipGraphDestroy(gr->graph);
			(void) hipGetLastError();
			g_pool.release_graph(&gr->blocks);
			if (graph == nullptr)
				throw Error(ERR_INVALID, "null output pointer");
			throw Error(ERR_DEVICE, std::string("the recording could not be turned into a graph: ") + hipGetErrorString(e));
		}
		gr->recorded_at = alloc_clock_tick();
		g_live_graphs.push_back(gr->recorded_at);
		*graph = reinterpret_cast<cattle_hip_graph_t>(gr.release());
	});
}

int cattle_hip_graph_launch(cattle_hip_graph_t graph) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(graph != nullptr, "null graph handle");
		forbid_while_capturing("launching a graph");
		g_deferred.settle();            /* the recorded calls did not know of sums that eager passes have left pending since */
		CATTLE_HIP_CHECK(hipGraphLaunch(reinterpret_cast<Graph*>(graph)->exec, stream()));
	});
}

int cattle_hip_graph_destroy(cattle_hip_graph_t graph) {
	return guarded([&] {
		if (!graph)
			return;
		forbid_while_capturing("destroying a graph");
		Graph* gr = reinterpret_cast<Graph*>(graph);
		CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
		(void) hipGraphExecDestroy(gr->exec);
		(void) hipGraphDestroy(gr->graph);
		g_pool.release_graph(&gr->blocks);
		std::vector<uint64_t>::iterator at = std::find(g_live_graphs.begin(), g_live_graphs.end(), gr->recorded_at);
		if (at != g_live_graphs.end())
			g_live_graphs.erase(at);
		free_unpinned_parked();
		delete gr;
	});
}

int cattle_hip_conv_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, size_t filters,
		size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_stride, size_t horizontal_stride, size_t vertical_dilation, size_t horizontal_dilation,
		cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr, "null output pointer");
		/* the constructor assertions of layer/kernel/ConvKernelLayer.hpp:82-87 */
		CATTLE_HIP_REQUIRE(height > 0 && width > 0 && channels > 0, "input dimensions must be positive");
		CATTLE_HIP_REQUIRE(filters > 0, "filters must be positive");
		CATTLE_HIP_REQUIRE(receptor_height > 0 && receptor_width > 0, "receptor dimensions must be positive");
		CATTLE_HIP_REQUIRE(vertical_stride > 0 && horizontal_stride > 0, "strides must be positive");
		const size_t lim = 1u << 20;
		CATTLE_HIP_REQUIRE(height < lim && width < lim && channels < lim && filters < lim && receptor_height < lim &&
				receptor_width < lim && vertical_padding < lim && horizontal_padding < lim && vertical_stride < lim &&
				horizontal_stride < lim && vertical_dilation < lim && horizontal_dilation < lim, "dimension too large");
		const size_t drh = receptor_height + (receptor_height - 1) * vertical_dilation;
		const size_t drw = receptor_width + (receptor_width - 1) * horizontal_dilation;
		CATTLE_HIP_REQUIRE(height + 2 * vertical_padding >= drh && width + 2 * horizontal_padding >= drw,
				"dilated receptor larger than the padded input");
		CATTLE_HIP_REQUIRE(receptor_height * receptor_width * channels <= 2147483647u / 2 &&
				receptor_height * receptor_width * filters <= 2147483647u / 2, "receptor volume too large");
		ConvShape s = { (int) height, (int) width, (int) channels, (int) filters, (int) receptor_height, (int) receptor_width,
				(int) vertical_padding, (int) horizontal_padding, (int) vertical_stride, (int) horizontal_stride,
				(int) vertical_dilation, (int) horizontal_dilation };
		LayerBase* l = dtype == CATTLE_HIP_F32 ? (LayerBase*) new ConvLayer<float>(dtype, s, false) :
				(LayerBase*) new ConvLayer<double>(dtype, s, false);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_conv_forward_noalloc(cattle_hip_dtype dtype, size_t batch, size_t height, size_t width, size_t channels,
		size_t filters, size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_stride, size_t horizontal_stride, size_t vertical_dilation, size_t horizontal_dilation,
		const void* in_device, const void* weights_device, const void* bias_device, void* out_device) {
	/* no allocation on this path: no layer object, no staging, no grow-only buffer; only kernel launches */
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(in_device != nullptr && weights_device != nullptr && out_device != nullptr, "null tensor buffer");
		CATTLE_HIP_REQUIRE(batch > 0 && batch <= 2147483647u, "batch size must be positive and below 2^31");
		CATTLE_HIP_REQUIRE(height > 0 && width > 0 && channels > 0 && filters > 0, "dimensions must be positive");
		CATTLE_HIP_REQUIRE(receptor_height > 0 && receptor_width > 0, "receptor dimensions must be positive");
		CATTLE_HIP_REQUIRE(vertical_stride > 0 && horizontal_stride > 0, "strides must be positive");
		const size_t lim = 1u << 20;
		CATTLE_HIP_REQUIRE(height < lim && width < lim && channels < lim && filters < lim && receptor_height < lim &&
				receptor_width < lim && vertical_padding < lim && horizontal_padding < lim && vertical_stride < lim &&
				horizontal_stride < lim && vertical_dilation < lim && horizontal_dilation < lim, "dimension too large");
		const size_t drh = receptor_height + (receptor_height - 1) * vertical_dilation;
		const size_t drw = receptor_width + (receptor_width - 1) * horizontal_dilation;
		CATTLE_HIP_REQUIRE(height + 2 * vertical_padding >= drh && width + 2 * horizontal_padding >= drw,
				"dilated receptor larger than the padded input");
		CATTLE_HIP_REQUIRE(receptor_height * receptor_width * channels <= 2147483647u / 2, "receptor volume too large");
		const ConvShape s = { (int) height, (int) width, (int) channels, (int) filters, (int) receptor_height, (int) receptor_width,
				(int) vertical_padding, (int) horizontal_padding, (int) vertical_stride, (int) horizontal_stride,
				(int) vertical_dilation, (int) horizontal_dilation };
		CATTLE_HIP_REQUIRE((double) batch * s.H * s.W * s.C <= 2147483647.0 && (double) batch * s.OH() * s.OW() * s.F <= 2147483647.0,
				"tensor exceeds 2^31-1 elements");
		if (dtype == CATTLE_HIP_F32)
			conv_forward_static<float>(s, (int) batch, static_cast<const float*>(in_device), static_cast<const float*>(weights_device),
					static_cast<const float*>(bias_device), static_cast<float*>(out_device));
		else
			conv_forward_static<double>(s, (int) batch, static_cast<const double*>(in_device),
					static_cast<const double*>(weights_device), static_cast<const double*>(bias_device), static_cast<double*>(out_device));
	});
}

int cattle_hip_static_scratch_bytes(size_t* bytes) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(bytes != nullptr, "null output pointer");
		*bytes = static_scratch_bytes();
	});
}

int cattle_hip_transconv_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, size_t filters,
		size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_stride, size_t horizontal_stride, size_t vertical_dilation, size_t horizontal_dilation,
		cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr, "null output pointer");
		/* the constructor assertions of layer/kernel/TransConvKernelLayer.hpp:84-89 */
		CATTLE_HIP_REQUIRE(height > 0 && width > 0 && channels > 0, "input dimensions must be positive");
		CATTLE_HIP_REQUIRE(filters > 0, "filters must be positive");
		CATTLE_HIP_REQUIRE(receptor_height > 0 && receptor_width > 0, "receptor dimensions must be positive");
		CATTLE_HIP_REQUIRE(vertical_stride > 0 && horizontal_stride > 0, "strides must be positive");
		const size_t lim = 1u << 20;
		CATTLE_HIP_REQUIRE(height < lim && width < lim && channels < lim && filters < lim && receptor_height < lim &&
				receptor_width < lim && vertical_padding < lim && horizontal_padding < lim && vertical_stride < lim &&
				horizontal_stride < lim && vertical_dilation < lim && horizontal_dilation < lim, "dimension too large");
		/* calculate_spatial_output_dim (:226-229) */
		const size_t drh = receptor_height + (receptor_height - 1) * vertical_dilation;
		const size_t drw = receptor_width + (receptor_width - 1) * horizontal_dilation;
		const size_t full_h = (height - 1) * vertical_stride + drh, full_w = (width - 1) * horizontal_stride + drw;
		CATTLE_HIP_REQUIRE(full_h > 2 * vertical_padding && full_w > 2 * horizontal_padding,
				"the padding cuts away the whole output");
		const size_t out_h = full_h - 2 * vertical_padding, out_w = full_w - 2 * horizontal_padding;
		CATTLE_HIP_REQUIRE(out_h < lim && out_w < lim, "dimension too large");
		CATTLE_HIP_REQUIRE(receptor_height * receptor_width * channels <= 2147483647u / 2 &&
				receptor_height * receptor_width * filters <= 2147483647u / 2, "receptor volume too large");
		/* the equivalent convolution maps the output (out_h, out_w, filters) back to the input */
		ConvShape c = { (int) out_h, (int) out_w, (int) filters, (int) channels, (int) receptor_height, (int) receptor_width,
				(int) vertical_padding, (int) horizontal_padding, (int) vertical_stride, (int) horizontal_stride,
				(int) vertical_dilation, (int) horizontal_dilation };
		if ((size_t) c.OH() != height || (size_t) c.OW() != width)
			throw Error(ERR_INVALID, "inconsistent transposed convolution geometry");
		LayerBase* l = dtype == CATTLE_HIP_F32 ? (LayerBase*) new TransConvLayer<float>(dtype, c) :
				(LayerBase*) new TransConvLayer<double>(dtype, c);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_convlstm_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, size_t hidden_channels,
		size_t receptor_height, size_t receptor_width, size_t vertical_padding, size_t horizontal_padding,
		size_t vertical_dilation, size_t horizontal_dilation, const int activation_kinds[5], const double activation_params[5],
		int foremost, cattle_hip_layer_t* lstm) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(lstm != nullptr && activation_kinds != nullptr, "null pointer argument");
		CATTLE_HIP_REQUIRE(height > 0 && width > 0 && channels > 0 && hidden_channels > 0, "dimensions must be positive");
		CATTLE_HIP_REQUIRE(receptor_height > 0 && receptor_width > 0, "receptor dimensions must be positive");
		const size_t lim = 1u << 20;
		CATTLE_HIP_REQUIRE(height < lim && width < lim && channels < lim && hidden_channels < lim / 4 && receptor_height < lim &&
				receptor_width < lim && vertical_padding < lim && horizontal_padding < lim && vertical_dilation < lim &&
				horizontal_dilation < lim, "dimension too large");
		CATTLE_HIP_REQUIRE(receptor_height * receptor_width * std::max(channels, hidden_channels) <= 2147483647u / 8,
				"receptor volume too large");
		for (int i = 0; i < 5; ++i)
			CATTLE_HIP_REQUIRE(activation_kinds[i] >= CATTLE_HIP_ACT_IDENTITY && activation_kinds[i] <= CATTLE_HIP_ACT_SWISH,
					"the cell's activations must be element-wise kinds");
		ConvShape x = { (int) height, (int) width, (int) channels, (int) (4 * hidden_channels), (int) receptor_height,
				(int) receptor_width, (int) vertical_padding, (int) horizontal_padding, 1, 1, (int) vertical_dilation,
				(int) horizontal_dilation };
		/* every kernel's output dims must be the state dims (LSTMNeuralNetwork.hpp:88-101) */
		const size_t drh = receptor_height + (receptor_height - 1) * vertical_dilation;
		const size_t drw = receptor_width + (receptor_width - 1) * horizontal_dilation;
		CATTLE_HIP_REQUIRE(height + 2 * vertical_padding >= drh && width + 2 * horizontal_padding >= drw &&
				(size_t) x.OH() == height && (size_t) x.OW() == width, "the kernels must keep the spatial dimensions");
		ConvShape h = x;
		h.C = (int) hidden_channels;
		LayerBase* l;
		if (dtype == CATTLE_HIP_F32) {
			LstmActs<float> a;
			for (int i = 0; i < 5; ++i) {
				a.kind[i] = activation_kinds[i];
				a.param[i] = activation_params ? (float) activation_params[i] : 0.0f;
			}
			l = new ConvLstm<float>(dtype, x, h, a, foremost != 0);
		} else {
			LstmActs<double> a;
			for (int i = 0; i < 5; ++i) {
				a.kind[i] = activation_kinds[i];
				a.param[i] = activation_params ? activation_params[i] : 0.0;
			}
			l = new ConvLstm<double>(dtype, x, h, a, foremost != 0);
		}
		*lstm = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_convlstm_propagate(cattle_hip_layer_t lstm, const void* input, cattle_hip_memspace input_space, size_t batch,
		size_t input_seq_length, size_t output_seq_length, size_t output_seq_delay, int training, void* out,
		cattle_hip_memspace out_space) {
	(void) training;        /* the caches a training pass needs are always kept */
	return guarded([&] {
		LayerBase* l = as_layer(lstm);
		check_space(input_space);
		check_space(out_space);
		CATTLE_HIP_REQUIRE(input != nullptr && out != nullptr, "null tensor buffer");
		CATTLE_HIP_REQUIRE(batch > 0 && input_seq_length > 0, "batch size and input sequence length must be positive");
		CATTLE_HIP_REQUIRE(output_seq_length > 0, "output sequence length must be positive");          /* :244 */
		if (ConvLstm<float>* f = dynamic_cast<ConvLstm<float>*>(l))
			convlstm_propagate<float>(f, input, input_space, batch, input_seq_length, output_seq_length, output_seq_delay, out,
					out_space);
		else if (ConvLstm<double>* d = dynamic_cast<ConvLstm<double>*>(l))
			convlstm_propagate<double>(d, input, input_space, batch, input_seq_length, output_seq_length, output_seq_delay, out,
					out_space);
		else
			throw Error(ERR_INVALID, "not a ConvLSTM handle");
	});
}

int cattle_hip_convlstm_backpropagate(cattle_hip_layer_t lstm, const void* out_grad, cattle_hip_memspace grad_space,
		void* in_grad, cattle_hip_memspace in_grad_space) {
	return guarded([&] {
		LayerBase* l = as_layer(lstm);
		check_space(grad_space);
		check_space(in_grad_space);
		CATTLE_HIP_REQUIRE(out_grad != nullptr, "null gradient buffer");
		ConvLstm<float>* f = dynamic_cast<ConvLstm<float>*>(l);
		ConvLstm<double>* d = dynamic_cast<ConvLstm<double>*>(l);
		CATTLE_HIP_REQUIRE(f || d, "not a ConvLSTM handle");
		const bool foremost = f ? f->foremost : d->foremost;
		CATTLE_HIP_REQUIRE(foremost == (in_grad == nullptr),
				"the input gradient buffer must be NULL exactly when the network is foremost");
		if (f)
			convlstm_backpropagate<float>(f, out_grad, grad_space, in_grad, in_grad_space);
		else
			convlstm_backpropagate<double>(d, out_grad, grad_space, in_grad, in_grad_space);
	});
}

int cattle_hip_convlstm_set_kernel_values(cattle_hip_layer_t lstm, size_t kernel, int bias, const void* values,
		cattle_hip_memspace space) {
	return guarded([&] {
		check_space(space);
		CATTLE_HIP_REQUIRE(values != nullptr, "null buffer");
		size_t offset, bytes;
		Param& p = lstm_kernel_param(lstm, kernel, bias, offset, bytes);
		copy_in((char*) p.values.p + offset, values, space, bytes);
		++p.version;
	});
}

int cattle_hip_convlstm_get_kernel_values(cattle_hip_layer_t lstm, size_t kernel, int bias, void* values,
		cattle_hip_memspace space) {
	return guarded([&] {
		check_space(space);
		CATTLE_HIP_REQUIRE(values != nullptr, "null buffer");
		size_t offset, bytes;
		Param& p = lstm_kernel_param(lstm, kernel, bias, offset, bytes);
		copy_out(values, space, (const char*) p.values.p + offset, bytes);
	});
}

int cattle_hip_convlstm_get_kernel_grad(cattle_hip_layer_t lstm, size_t kernel, int bias, void* grad, cattle_hip_memspace space) {
	return guarded([&] {
		check_space(space);
		CATTLE_HIP_REQUIRE(grad != nullptr, "null buffer");
		size_t offset, bytes;
		Param& p = lstm_kernel_param(lstm, kernel, bias, offset, bytes);
		g_deferred.settle();
		copy_out(grad, space, (const char*) p.grad.p + offset, bytes);
	});
}

int cattle_hip_convlstm_set_multiplicative_integration(cattle_hip_layer_t lstm, int enabled) {
	return guarded([&] {
		LayerBase* l = as_layer(lstm);
		ConvLstm<float>* f = dynamic_cast<ConvLstm<float>*>(l);
		ConvLstm<double>* d = dynamic_cast<ConvLstm<double>*>(l);
		CATTLE_HIP_REQUIRE(f || d, "not a ConvLSTM handle");
		(f ? f->mul_int : d->mul_int) = enabled != 0;
		l->empty_cache();           /* the caches of a pass made under the other rule do not fit this one */
	});
}

int cattle_hip_convlstm_fused_steps(cattle_hip_layer_t lstm, int* forward_steps, int* backward_steps) {
	return guarded([&] {
		LayerBase* l = as_layer(lstm);
		ConvLstm<float>* f = dynamic_cast<ConvLstm<float>*>(l);
		ConvLstm<double>* d = dynamic_cast<ConvLstm<double>*>(l);
		CATTLE_HIP_REQUIRE(f || d, "not a ConvLSTM handle");
		CATTLE_HIP_REQUIRE(forward_steps != nullptr && backward_steps != nullptr, "null output pointer");
		*forward_steps = f ? f->fused_forward_steps : d->fused_forward_steps;
		*backward_steps = f ? f->fused_backward_steps : d->fused_backward_steps;
	});
}

int cattle_hip_dense_create(cattle_hip_dtype dtype, size_t input_volume, size_t output_size, cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr, "null output pointer");
		CATTLE_HIP_REQUIRE(input_volume > 0 && output_size > 0, "dense layer sizes must be positive");
		CATTLE_HIP_REQUIRE(input_volume <= 2147483647u / 2 && output_size <= 2147483647u / 2, "dense layer too large");
		ConvShape s = { 1, 1, (int) input_volume, (int) output_size, 1, 1, 0, 0, 1, 1, 0, 0 };
		LayerBase* l = dtype == CATTLE_HIP_F32 ? (LayerBase*) new ConvLayer<float>(dtype, s, true) :
				(LayerBase*) new ConvLayer<double>(dtype, s, true);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_batchnorm_create(cattle_hip_dtype dtype, size_t height, size_t width, size_t channels, int per_last_rank,
		double norm_avg_decay, double epsilon, cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr, "null output pointer");
		CATTLE_HIP_REQUIRE(height > 0 && width > 0 && channels > 0, "dimensions must be positive");
		/* layer/BatchNormLayer.hpp:80-82 */
		CATTLE_HIP_REQUIRE(norm_avg_decay >= 0 && norm_avg_decay <= 1, "norm avg decay must not be less than 0 or greater than 1");
		CATTLE_HIP_REQUIRE(epsilon > 0, "epsilon must be greater than 0");
		LayerBase* l = dtype == CATTLE_HIP_F32 ?
				(LayerBase*) new BatchNormLayer<float>(dtype, height, width, channels, per_last_rank != 0, (float) norm_avg_decay,
						(float) epsilon) :
				(LayerBase*) new BatchNormLayer<double>(dtype, height, width, channels, per_last_rank != 0, norm_avg_decay, epsilon);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_batchnorm_get_stats_initialized(cattle_hip_layer_t layer, int* initialized) {
	return guarded([&] {
		LayerBase* l = as_layer(layer);
		CATTLE_HIP_REQUIRE(initialized != nullptr, "null output pointer");
		if (BatchNormLayer<float>* b = dynamic_cast<BatchNormLayer<float>*>(l))
			*initialized = b->stats_init;
		else if (BatchNormLayer<double>* b = dynamic_cast<BatchNormLayer<double>*>(l))
			*initialized = b->stats_init;
		else
			throw Error(ERR_INVALID, "not a batch norm layer");
	});
}

int cattle_hip_batchnorm_set_stats_initialized(cattle_hip_layer_t layer, int initialized) {
	return guarded([&] {
		LayerBase* l = as_layer(layer);
		if (BatchNormLayer<float>* b = dynamic_cast<BatchNormLayer<float>*>(l))
			b->stats_init = initialized != 0;
		else if (BatchNormLayer<double>* b = dynamic_cast<BatchNormLayer<double>*>(l))
			b->stats_init = initialized != 0;
		else
			throw Error(ERR_INVALID, "not a batch norm layer");
	});
}

int cattle_hip_activation_create(cattle_hip_dtype dtype, cattle_hip_activation kind, size_t volume, double param,
		cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr, "null output pointer");
		CATTLE_HIP_REQUIRE(volume > 0, "volume must be positive");
		CATTLE_HIP_REQUIRE((int) kind >= 0 && (int) kind <= CATTLE_HIP_ACT_PSWISH, "unknown activation kind");
		LayerBase* l = dtype == CATTLE_HIP_F32 ? (LayerBase*) new ActivationLayer<float>(dtype, kind, volume, (float) param) :
				(LayerBase*) new ActivationLayer<double>(dtype, kind, volume, param);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_pool_create(cattle_hip_dtype dtype, cattle_hip_pool kind, size_t height, size_t width, size_t channels,
		size_t receptor_height, size_t receptor_width, size_t vertical_stride, size_t horizontal_stride,
		cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr, "null output pointer");
		CATTLE_HIP_REQUIRE(kind == CATTLE_HIP_POOL_MAX || kind == CATTLE_HIP_POOL_MEAN, "unknown pool kind");
		/* layer/PoolLayer.hpp:73-75 */
		CATTLE_HIP_REQUIRE(receptor_height > 0 && receptor_width > 0, "receptor dimensions must be positive");
		CATTLE_HIP_REQUIRE(vertical_stride > 0 && horizontal_stride > 0, "strides must be positive");
		CATTLE_HIP_REQUIRE(channels > 0 && height >= receptor_height && width >= receptor_width, "receptor larger than the input");
		const size_t lim = 1u << 20;
		CATTLE_HIP_REQUIRE(height < lim && width < lim && channels < lim && vertical_stride < lim && horizontal_stride < lim,
				"dimension too large");
		CATTLE_HIP_REQUIRE(receptor_height * receptor_width < 65536, "receptor area too large");
		PoolShape s = { (int) height, (int) width, (int) channels, (int) receptor_height, (int) receptor_width,
				(int) vertical_stride, (int) horizontal_stride };
		LayerBase* l = dtype == CATTLE_HIP_F32 ? (LayerBase*) new PoolLayer<float>(dtype, kind, s) :
				(LayerBase*) new PoolLayer<double>(dtype, kind, s);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_fused_create(const cattle_hip_layer_t* layers, size_t count, cattle_hip_layer_t* fused) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(layers != nullptr && fused != nullptr, "null pointer");
		CATTLE_HIP_REQUIRE(count >= 1 && count <= 4, "a fused layer has one to four members");
		std::vector<LayerBase*> members;
		for (size_t i = 0; i < count; ++i) {
			members.push_back(as_layer(layers[i]));
			CATTLE_HIP_REQUIRE(members[i]->dtype == members[0]->dtype, "members differ in scalar type");
			for (size_t j = 0; j < i; ++j)
				CATTLE_HIP_REQUIRE(members[j] != members[i], "a layer is listed twice");
		}
		LayerBase* l = members[0]->dtype == CATTLE_HIP_F32 ? (LayerBase*) new FusedLayer<float>(CATTLE_HIP_F32, members, false) :
				(LayerBase*) new FusedLayer<double>(CATTLE_HIP_F64, members, false);
		*fused = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_fused_last_mode(cattle_hip_layer_t fused, int* mode) {
	return guarded([&] {
		LayerBase* l = as_layer(fused);
		CATTLE_HIP_REQUIRE(mode != nullptr, "null output pointer");
		if (FusedLayer<float>* f = dynamic_cast<FusedLayer<float>*>(l))
			*mode = f->mode;
		else if (FusedLayer<double>* f = dynamic_cast<FusedLayer<double>*>(l))
			*mode = f->mode;
		else
			throw Error(ERR_INVALID, "not a fused layer");
	});
}

int cattle_hip_dropout_create(cattle_hip_dtype dtype, size_t volume, double dropout_prob, double epsilon, unsigned long long seed,
		cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr, "null output pointer");
		CATTLE_HIP_REQUIRE(volume > 0, "volume must be positive");
		/* layer/DropoutLayer.hpp:39-41 */
		CATTLE_HIP_REQUIRE(dropout_prob > 0 && dropout_prob <= 1, "dropout probability must be greater than 0 and no greater than 1");
		CATTLE_HIP_REQUIRE(epsilon > 0, "epsilon must be greater than 0");
		LayerBase* l = dtype == CATTLE_HIP_F32 ?
				(LayerBase*) new DropoutLayer<float>(dtype, volume, (float) dropout_prob, (float) epsilon, seed) :
				(LayerBase*) new DropoutLayer<double>(dtype, volume, dropout_prob, epsilon, seed);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_reshape_create(cattle_hip_dtype dtype, const size_t input_dims[3], const size_t output_dims[3],
		cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr && input_dims != nullptr && output_dims != nullptr, "null pointer");
		const size_t lim = 2147483647u;
		for (int i = 0; i < 3; ++i)
			CATTLE_HIP_REQUIRE(input_dims[i] > 0 && output_dims[i] > 0 && input_dims[i] <= lim && output_dims[i] <= lim,
					"dimensions must be positive and below 2^31");
		CATTLE_HIP_REQUIRE(input_dims[0] * input_dims[1] <= lim / input_dims[2] &&
				output_dims[0] * output_dims[1] <= lim / output_dims[2], "volume exceeds 2^31-1");
		/* layer/ReshapeLayer.hpp:38 */
		CATTLE_HIP_REQUIRE(input_dims[0] * input_dims[1] * input_dims[2] == output_dims[0] * output_dims[1] * output_dims[2],
				"the input and output volumes differ");
		*layer = reinterpret_cast<cattle_hip_layer_t>((LayerBase*) new ReshapeLayer(dtype, input_dims, output_dims));
	});
}

int cattle_hip_broadcast_create(cattle_hip_dtype dtype, const size_t input_dims[3], const size_t broadcast[3],
		cattle_hip_layer_t* layer) {
	return guarded([&] {
		check_dtype(dtype);
		CATTLE_HIP_REQUIRE(layer != nullptr && input_dims != nullptr && broadcast != nullptr, "null pointer");
		const size_t lim = 2147483647u;
		size_t volume = 1;
		for (int i = 0; i < 3; ++i) {
			/* layer/BroadcastLayer.hpp:38-39 */
			CATTLE_HIP_REQUIRE(input_dims[i] > 0 && broadcast[i] > 0, "dimensions and repetitions must be positive");
			CATTLE_HIP_REQUIRE(input_dims[i] <= lim && broadcast[i] <= lim / input_dims[i] &&
					input_dims[i] * broadcast[i] <= lim / volume, "output volume exceeds 2^31-1");
			volume *= input_dims[i] * broadcast[i];
		}
		LayerBase* l = dtype == CATTLE_HIP_F32 ? (LayerBase*) new BroadcastLayer<float>(dtype, input_dims, broadcast) :
				(LayerBase*) new BroadcastLayer<double>(dtype, input_dims, broadcast);
		*layer = reinterpret_cast<cattle_hip_layer_t>(l);
	});
}

int cattle_hip_layer_clone(cattle_hip_layer_t layer, int share_params, cattle_hip_layer_t* clone) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(clone != nullptr, "null output pointer");
		g_deferred.settle();            /* a deep copy copies the gradients */
		*clone = reinterpret_cast<cattle_hip_layer_t>(as_layer(layer)->clone(share_params != 0));
	});
}

int cattle_hip_layer_destroy(cattle_hip_layer_t layer) {
	return guarded([&] {
		if (layer) {
			forbid_while_capturing("waiting for the device");
			g_deferred.settle();        /* partial sums of a bias gradient lie in the buffer of the weights' parameter object */
			CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
			delete reinterpret_cast<LayerBase*>(layer);
		}
	});
}

int cattle_hip_layer_input_dims(cattle_hip_layer_t layer, size_t dims[3]) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(dims != nullptr, "null output pointer");
		std::memcpy(dims, as_layer(layer)->in_dims, 3 * sizeof(size_t));
	});
}

int cattle_hip_layer_output_dims(cattle_hip_layer_t layer, size_t dims[3]) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(dims != nullptr, "null output pointer");
		std::memcpy(dims, as_layer(layer)->out_dims, 3 * sizeof(size_t));
	});
}

int cattle_hip_layer_is_input_layer(cattle_hip_layer_t layer, int* is_input_layer) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(is_input_layer != nullptr, "null output pointer");
		*is_input_layer = as_layer(layer)->input_layer ? 1 : 0;
	});
}

int cattle_hip_layer_set_input_layer(cattle_hip_layer_t layer, int is_input_layer) {
	return guarded([&] { as_layer(layer)->input_layer = is_input_layer != 0; });
}

int cattle_hip_layer_empty_cache(cattle_hip_layer_t layer) {
	return guarded([&] {
		forbid_while_capturing("waiting for the device");
		/* the caches it frees may be what a living graph, recorded after the layer was created, points into */
		if (pinned_by_graph(as_layer(layer)->created))
			throw Error(ERR_STATE, "a recorded graph may point into the layer's caches: destroy the graph (cattle_hip_graph_destroy) "
					"before emptying them");
		CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
		as_layer(layer)->empty_cache();
	});
}

int cattle_hip_layer_forward(cattle_hip_layer_t layer, const void* in, cattle_hip_memspace in_space, size_t batch,
		int training, void* out, cattle_hip_memspace out_space) {
	return guarded([&] {
		LayerBase* l = as_layer(layer);
		check_space(in_space);
		check_space(out_space);
		CATTLE_HIP_REQUIRE(in != nullptr && out != nullptr, "null tensor buffer");
		CATTLE_HIP_REQUIRE(batch > 0, "batch size must be positive");            /* assert(in.dimension(0) > 0) */
		const size_t in_bytes = batch * l->in_volume() * l->esize(), out_bytes = batch * l->out_volume() * l->esize();
		CATTLE_HIP_REQUIRE(batch * l->in_volume() <= 2147483647u && batch * l->out_volume() <= 2147483647u,
				"tensor exceeds 2^31-1 elements");
		const void* in_dev = in;
		if (in_space == CATTLE_HIP_HOST) {
			copy_in(l->in_stage.ensure(in_bytes), in, CATTLE_HIP_HOST, in_bytes);
			in_dev = l->in_stage.p;
		}
		void* out_dev = out_space == CATTLE_HIP_HOST ? l->out_stage.ensure(out_bytes) : out;
		l->have_forward = false;
		l->forward(in_dev, batch, training != 0, out_dev);
		if (out_space == CATTLE_HIP_HOST)
			copy_out(out, CATTLE_HIP_HOST, out_dev, out_bytes);
		l->batch = batch;
		l->have_forward = true;
	});
}

int cattle_hip_layer_backward(cattle_hip_layer_t layer, const void* out_grad, cattle_hip_memspace grad_space, size_t batch,
		void* in_grad, cattle_hip_memspace in_grad_space) {
	return guarded([&] {
		LayerBase* l = as_layer(layer);
		check_space(grad_space);
		check_space(in_grad_space);
		CATTLE_HIP_REQUIRE(out_grad != nullptr, "null gradient buffer");
		if (!l->have_forward)
			throw Error(ERR_STATE, "pass_back without a preceding pass_forward");
		CATTLE_HIP_REQUIRE(batch > 0 && batch == l->batch, "batch size differs from the forward pass");   /* e.g. ConvKernelLayer.hpp:314 */
		CATTLE_HIP_REQUIRE(in_grad != nullptr || l->input_layer, "in_grad may be NULL only for an input layer");
		l->check_borrowed();
		const size_t in_bytes = batch * l->in_volume() * l->esize(), out_bytes = batch * l->out_volume() * l->esize();
		const void* og_dev = out_grad;
		if (grad_space == CATTLE_HIP_HOST) {
			copy_in(l->og_stage.ensure(out_bytes), out_grad, CATTLE_HIP_HOST, out_bytes);
			og_dev = l->og_stage.p;
		}
		const bool want_in_grad = in_grad != nullptr && (!l->input_layer || l->always_backprop);
		void* ig_dev = nullptr;
		if (want_in_grad)
			ig_dev = in_grad_space == CATTLE_HIP_HOST ? l->ig_stage.ensure(in_bytes) : in_grad;
		l->backward(og_dev, batch, ig_dev);
		/* accumulate_grad enforces the gradient's constraints after every accumulation (StandardParameters.hpp:119-122) */
		for (const ParamPtr& q : l->params)
			if (q->optimizable && q->constrains_grad()) {
				g_deferred.settle();
				constrain(*q, false);
			}
		if (want_in_grad && in_grad_space == CATTLE_HIP_HOST)
			copy_out(in_grad, CATTLE_HIP_HOST, ig_dev, in_bytes);
	});
}

int cattle_hip_layer_num_params(cattle_hip_layer_t layer, size_t* count) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(count != nullptr, "null output pointer");
		*count = as_layer(layer)->params.size();
	});
}

int cattle_hip_layer_param_shape(cattle_hip_layer_t layer, size_t index, size_t* rows, size_t* cols, int* optimizable) {
	return guarded([&] {
		Param& p = param_at(as_layer(layer), index);
		if (rows)
			*rows = p.rows;
		if (cols)
			*cols = p.cols;
		if (optimizable)
			*optimizable = p.optimizable ? 1 : 0;
	});
}

int cattle_hip_layer_set_param_values(cattle_hip_layer_t layer, size_t index, const void* values, cattle_hip_memspace space) {
	return guarded([&] {
		check_space(space);
		CATTLE_HIP_REQUIRE(values != nullptr, "null buffer");
		Param& p = param_at(as_layer(layer), index);
		copy_in(p.values.p, values, space, p.bytes());
		if (p.constrains_values())
			constrain(p, true);
		++p.version;
	});
}

int cattle_hip_layer_get_param_values(cattle_hip_layer_t layer, size_t index, void* values, cattle_hip_memspace space) {
	return guarded([&] {
		check_space(space);
		CATTLE_HIP_REQUIRE(values != nullptr, "null buffer");
		Param& p = param_at(as_layer(layer), index);
		copy_out(values, space, p.values.p, p.bytes());
	});
}

int cattle_hip_layer_get_param_grad(cattle_hip_layer_t layer, size_t index, void* grad, cattle_hip_memspace space) {
	return guarded([&] {
		check_space(space);
		CATTLE_HIP_REQUIRE(grad != nullptr, "null buffer");
		Param& p = param_at(as_layer(layer), index);
		g_deferred.settle();
		copy_out(grad, space, p.grad.p, p.bytes());
	});
}

int cattle_hip_layer_reset_param_grad(cattle_hip_layer_t layer, size_t index) {
	return guarded([&] {
		Param& p = param_at(as_layer(layer), index);
		g_deferred.settle();
		fill_zero(p.grad.p, p.bytes());
	});
}

int cattle_hip_loss_function(cattle_hip_dtype dtype, cattle_hip_loss kind, const void* out, cattle_hip_memspace out_space,
		const void* obj, cattle_hip_memspace obj_space, size_t batch, size_t time_steps, size_t sample_size,
		double epsilon, void* losses, cattle_hip_memspace losses_space) {
	return guarded([&] {
		loss_entry(false, dtype, kind, out, out_space, obj, obj_space, batch, time_steps, sample_size, epsilon, 1.0, losses,
				losses_space);
	});
}

int cattle_hip_loss_d_function(cattle_hip_dtype dtype, cattle_hip_loss kind, const void* out, cattle_hip_memspace out_space,
		const void* obj, cattle_hip_memspace obj_space, size_t batch, size_t time_steps, size_t sample_size,
		double epsilon, double scale, void* grad, cattle_hip_memspace grad_space) {
	return guarded([&] {
		loss_entry(true, dtype, kind, out, out_space, obj, obj_space, batch, time_steps, sample_size, epsilon, scale, grad,
				grad_space);
	});
}

int cattle_hip_layer_param_optimizer_update(cattle_hip_layer_t layer, size_t index, cattle_hip_optimizer optimizer,
		const double hyper[4], size_t epoch, size_t timestep) {
	return guarded([&] { run_optimizer(layer, index, optimizer, hyper, epoch, timestep, false); });
}

int cattle_hip_layer_param_optimizer_step(cattle_hip_layer_t layer, size_t index, cattle_hip_optimizer optimizer,
		const double hyper[4], size_t epoch, size_t timestep) {
	return guarded([&] { run_optimizer(layer, index, optimizer, hyper, epoch, timestep, true); });
}

int cattle_hip_layer_param_set_regularization(cattle_hip_layer_t layer, size_t index, double l1_lambda, double l2_lambda) {
	return guarded([&] {
		Param& p = optimizable_param(layer, index);
		CATTLE_HIP_REQUIRE(l1_lambda == l1_lambda && l2_lambda == l2_lambda, "lambda is not a number");
		p.reg_l1 = l1_lambda;
		p.reg_l2 = l2_lambda;
	});
}

int cattle_hip_layer_param_set_constraints(cattle_hip_layer_t layer, size_t index, double value_clip, double value_max_l1_norm,
		double value_max_l2_norm, double grad_clip, double grad_max_l1_norm, double grad_max_l2_norm) {
	return guarded([&] {
		LayerBase* l = as_layer(layer);
		Param& p = param_at(l, index);
		const double v[6] = { value_clip, value_max_l1_norm, value_max_l2_norm, grad_clip, grad_max_l1_norm, grad_max_l2_norm };
		for (int i = 0; i < 6; ++i)
			CATTLE_HIP_REQUIRE(v[i] == v[i], "a limit is not a number");
		CATTLE_HIP_REQUIRE(dynamic_cast<ConvLstm<float>*>(l) == nullptr && dynamic_cast<ConvLstm<double>*>(l) == nullptr,
				"the fused LSTM accumulates the gradients of all time steps at once: constraints per accumulation cannot be enforced");
		std::memcpy(p.value_limits, v, sizeof(p.value_limits));
		std::memcpy(p.grad_limits, v + 3, sizeof(p.grad_limits));
		if (p.constrains_values()) {
			constrain(p, true);
			++p.version;
		}
	});
}

int cattle_hip_layer_param_regularization_penalty(cattle_hip_layer_t layer, size_t index, double* penalty) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(penalty != nullptr, "null output pointer");
		Param& p = param_at(as_layer(layer), index);
		*penalty = 0;
		if (!p.optimizable || (p.reg_l1 == 0 && p.reg_l2 == 0))        /* StandardParameters.hpp:128-132 */
			return;
		static DevBuf sums;
		sums.ensure(2 * sizeof(double));
		if (p.esize == sizeof(float)) {
			float h[2];
			regularization_sums<float>(p.rows * p.cols, static_cast<const float*>(p.values.p), static_cast<float*>(sums.p));
			copy_out(h, CATTLE_HIP_HOST, sums.p, sizeof(h));
			/* in the parameter's scalar type, as the reference computes it */
			const float l1 = (float) p.reg_l1, l2 = (float) p.reg_l2;
			*penalty = (double) ((l1 != 0 ? h[0] * l1 : 0.0f) + (l2 != 0 ? h[1] * (0.5f * l2) : 0.0f));
			return;
		}
		double h[2];
		regularization_sums<double>(p.rows * p.cols, static_cast<const double*>(p.values.p), static_cast<double*>(sums.p));
		copy_out(h, CATTLE_HIP_HOST, sums.p, sizeof(h));
		*penalty = (p.reg_l1 != 0 ? h[0] * p.reg_l1 : 0.0) + (p.reg_l2 != 0 ? h[1] * (0.5 * p.reg_l2) : 0.0);
	});
}

int cattle_hip_optimizer_step_many(const cattle_hip_layer_t* layers, const size_t* indices, size_t count,
		cattle_hip_optimizer optimizer, const double hyper[4], size_t epoch, size_t timestep) {
	return guarded([&] {
		CATTLE_HIP_REQUIRE(count == 0 || (layers != nullptr && indices != nullptr), "null parameter list");
		CATTLE_HIP_REQUIRE(hyper != nullptr, "null hyper-parameter array");
		if (count == 0)
			return;
		if (as_layer(layers[0])->dtype == CATTLE_HIP_F32)
			run_optimizer_many<float>(layers, indices, count, optimizer, hyper, epoch, timestep);
		else
			run_optimizer_many<double>(layers, indices, count, optimizer, hyper, epoch, timestep);
	});
}

int cattle_hip_layer_param_sgd_update(cattle_hip_layer_t layer, size_t index, double learning_rate) {
	const double hyper[4] = { learning_rate, 0, 0, 0 };
	return cattle_hip_layer_param_optimizer_update(layer, index, CATTLE_HIP_OPT_VANILLA_SGD, hyper, 0, 0);
}

int cattle_hip_layer_param_adam_update(cattle_hip_layer_t layer, size_t index, double learning_rate, double l1_decay,
		double l2_decay, double epsilon, size_t timestep) {
	const double hyper[4] = { learning_rate, l1_decay, l2_decay, epsilon };
	return cattle_hip_layer_param_optimizer_update(layer, index, CATTLE_HIP_OPT_ADAM, hyper, 0, timestep);
}

int cattle_hip_layer_param_reset_optimizer_state(cattle_hip_layer_t layer, size_t index) {
	return guarded([&] {
		Param& p = param_at(as_layer(layer), index);
		for (int i = 0; i < p.moments_ready; ++i)
			fill_zero(p.moments[i].p, p.bytes());
	});
}

int cattle_hip_maxpool_indices(cattle_hip_layer_t layer, unsigned* indices, cattle_hip_memspace space) {
	return guarded([&] {
		check_space(space);
		CATTLE_HIP_REQUIRE(indices != nullptr, "null buffer");
		LayerBase* l = as_layer(layer);
		DevBuf* buf = nullptr;
		size_t count = 0;
		if (PoolLayer<float>* p = dynamic_cast<PoolLayer<float>*>(l)) {
			buf = &p->inds;
			count = p->kind == CATTLE_HIP_POOL_MAX ? p->inds_count : 0;
		} else if (PoolLayer<double>* p = dynamic_cast<PoolLayer<double>*>(l)) {
			buf = &p->inds;
			count = p->kind == CATTLE_HIP_POOL_MAX ? p->inds_count : 0;
		}
		if (!buf || count == 0)
			throw Error(ERR_STATE, "no max-pool index cache (not a max pool layer, or no forward pass yet)");
		copy_out(indices, space, buf->p, count * sizeof(unsigned));
	});
}

} /* extern "C" */
