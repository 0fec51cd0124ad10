/*
 * host_copy.hip — copies between pageable host memory and the device.
 *
 * The tensors that cross the Layer API (core/Layer.hpp:126,137) are Eigen tensors in ordinary heap memory; they
 * cannot be allocated pinned through that API. A hipMemcpy from or to such memory is staged by the runtime on
 * one thread and reaches 17-28 GB/s on MI355X hosts, a third to a half of what the link carries from pinned
 * memory (57 GB/s). Large copies are therefore staged here: the tensor is cut into chunks, a few host threads
 * copy a chunk between the caller's memory and one of several pinned buffers while the DMA engine moves the
 * chunks before it, and events keep a buffer from being reused before its transfer is done. Measured: 50 GB/s in
 * both directions with four threads.
 *
 * The worker threads and the pinned buffers are created on the first large copy and live until the process
 * ends (they are never joined or freed: a static destructor could run after the HIP runtime has shut down).
 * Calls into the library are serialised by its caller-side lock, so there is one copy at a time.
 */
#include "common.hpp"

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <unistd.h>
#include <vector>

namespace cattle_hip {

namespace {

constexpr size_t STAGE_CHUNK = (size_t) 16 << 20;      /* bytes per pinned buffer */
constexpr int STAGE_BUFFERS = 4;
constexpr size_t STAGE_MIN_BYTES = (size_t) 4 << 20;   /* smaller copies go straight to the runtime */

/* memcpy of one range by several threads. The calling thread takes the first slice; workers sleep between jobs. */
struct CopyPool {
	std::mutex m;
	std::condition_variable wake, done;
	std::vector<std::thread> workers;
	char* dst = nullptr;
	const char* src = nullptr;
	size_t bytes = 0, slice = 0;
	unsigned long generation = 0;
	int pending = 0;
	pid_t owner;            /* threads do not survive fork(): a child process copies on its own thread */

	explicit CopyPool(int threads) : owner(getpid()) {
		for (int i = 1; i < threads; ++i)
			workers.emplace_back([this, i] { run(i); });
		for (std::thread& t : workers)
			t.detach();
	}
	void run(int index) {
		unsigned long seen = 0;
		for (;;) {
			char* d;
			const char* s;
			size_t n, per;
			{
				std::unique_lock<std::mutex> lock(m);
				wake.wait(lock, [&] { return generation != seen; });
				seen = generation;
				d = dst; s = src; n = bytes; per = slice;
			}
			const size_t begin = (size_t) index * per;
			if (begin < n)
				std::memcpy(d + begin, s + begin, std::min(per, n - begin));
			{
				std::lock_guard<std::mutex> lock(m);
				if (--pending == 0)
					done.notify_one();
			}
		}
	}
	void copy(void* d, const void* s, size_t n) {
		const int threads = (int) workers.size() + 1;
		if (threads == 1 || n < ((size_t) 1 << 20) || getpid() != owner) {
			std::memcpy(d, s, n);
			return;
		}
		const size_t per = ((n + threads - 1) / threads + 63) / 64 * 64;
		{
			std::lock_guard<std::mutex> lock(m);
			dst = static_cast<char*>(d);
			src = static_cast<const char*>(s);
			bytes = n;
			slice = per;
			pending = threads - 1;
			++generation;
		}
		wake.notify_all();
		std::memcpy(d, s, std::min(per, n));
		std::unique_lock<std::mutex> lock(m);
		done.wait(lock, [&] { return pending == 0; });
	}
};

struct Stager {
	char* buf[STAGE_BUFFERS];
	hipEvent_t ev[STAGE_BUFFERS];
	CopyPool* pool;
};

/* nullptr when staging is switched off (CATTLE_HIP_COPY_THREADS=0) */
Stager* stager() {
	static Stager* s = [] () -> Stager* {
		int threads = 4;
		if (const char* e = std::getenv("CATTLE_HIP_COPY_THREADS"))
			threads = std::atoi(e);
		if (threads <= 0)
			return nullptr;
		threads = std::min(threads, 16);
		Stager* st = new Stager();
		for (int i = 0; i < STAGE_BUFFERS; ++i) {
			CATTLE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&st->buf[i]), STAGE_CHUNK, hipHostMallocDefault));
			CATTLE_HIP_CHECK(hipEventCreateWithFlags(&st->ev[i], hipEventDisableTiming));
		}
		st->pool = new CopyPool(threads);
		return st;
	}();
	return s;
}

} /* namespace */

void host_to_device(void* dst_dev, const void* src_host, size_t bytes) {
	forbid_while_capturing("a copy between host and device memory");
	if (bytes == 0)
		return;
	Stager* st = bytes >= STAGE_MIN_BYTES ? stager() : nullptr;
	if (!st) {
		CATTLE_HIP_CHECK(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, stream()));
		CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));        /* the pageable source may be freed on return */
		return;
	}
	const char* src = static_cast<const char*>(src_host);
	char* dst = static_cast<char*>(dst_dev);
	int k = 0;
	for (size_t off = 0; off < bytes; off += STAGE_CHUNK, ++k) {
		const size_t n = std::min(STAGE_CHUNK, bytes - off);
		const int b = k % STAGE_BUFFERS;
		if (k >= STAGE_BUFFERS)
			CATTLE_HIP_CHECK(hipEventSynchronize(st->ev[b]));    /* the transfer that last used this buffer is done */
		st->pool->copy(st->buf[b], src + off, n);
		CATTLE_HIP_CHECK(hipMemcpyAsync(dst + off, st->buf[b], n, hipMemcpyHostToDevice, stream()));
		CATTLE_HIP_CHECK(hipEventRecord(st->ev[b], stream()));
	}
	/* the source has been read completely; the pinned buffers must not be refilled by a later call before their
	 * transfers are done, so wait for them here (a few chunks at link speed) */
	CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
}

void device_to_host(void* dst_host, const void* src_dev, size_t bytes) {
	forbid_while_capturing("a copy between host and device memory");
	if (bytes == 0)
		return;
	Stager* st = bytes >= STAGE_MIN_BYTES ? stager() : nullptr;
	if (!st) {
		CATTLE_HIP_CHECK(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, stream()));
		CATTLE_HIP_CHECK(hipStreamSynchronize(stream()));
		return;
	}
	char* dst = static_cast<char*>(dst_host);
	const char* src = static_cast<const char*>(src_dev);
	const size_t chunks = (bytes + STAGE_CHUNK - 1) / STAGE_CHUNK;
	/* transfers run STAGE_BUFFERS chunks ahead of the host-side copies */
	for (size_t k = 0; k < chunks + STAGE_BUFFERS; ++k) {
		const int b = (int) (k % STAGE_BUFFERS);
		if (k >= STAGE_BUFFERS) {
			const size_t off = (k - STAGE_BUFFERS) * STAGE_CHUNK;
			CATTLE_HIP_CHECK(hipEventSynchronize(st->ev[b]));
			st->pool->copy(dst + off, st->buf[b], std::min(STAGE_CHUNK, bytes - off));
		}
		if (k < chunks) {
			const size_t off = k * STAGE_CHUNK;
			CATTLE_HIP_CHECK(hipMemcpyAsync(st->buf[b], src + off, std::min(STAGE_CHUNK, bytes - off), hipMemcpyDeviceToHost,
					stream()));
			CATTLE_HIP_CHECK(hipEventRecord(st->ev[b], stream()));
		}
	}
}

} /* namespace cattle_hip */
