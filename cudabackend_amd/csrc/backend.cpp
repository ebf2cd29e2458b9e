/*
 * backend.cpp -- host side of the backend: descriptor store, argument validation, dispatch, status mapping.
 *
 * Takes the place of the reference's descriptor glue and entry points (src/descriptors.cu:48-322, src/cuda_properties.cpp,
 * src/utilities.hpp:23-58, and the `cuda*` entry functions at the bottom of src/winograd_nonfused.cu, src/gemm.cpp,
 * src/tensor_op.cu, src/im2row.cu, src/conversions.cu, src/convolution.cu, src/winograd_fused.cu,
 * src/conv2d_implicit_gemm.cu).  All device work goes through the C-ABI launchers of avocado_hip_kernels.h.
 *
 * Handles are 64-bit integers: bits 48..55 hold the descriptor kind, bits 32..47 the device, bits 0..31 a slot in a
 * per-kind table.  The default context of device d is the handle (kind = context, device = d, slot = 0xFFFFFFFF); it maps
 * to the null stream and, as in the reference (src/descriptors.cu:120-124), makes copies synchronous.
 *
 * Owning memory blocks keep a short log of the byte ranges that API calls wrote to them.  The cache of Winograd-transformed
 * weights reads it, so a weight tensor is re-transformed exactly when its own bytes were written since the cached copy was made.
 */
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

#include "../../include/avocado_hip_backend.h"
#include "../../include/avocado_hip_kernels.h"

namespace
{
	using namespace avocado::backend;

	enum Kind
	{
		KIND_CONTEXT = 1, KIND_MEMORY, KIND_TENSOR, KIND_CONVOLUTION
	};
	constexpr uint32_t DEFAULT_SLOT = 0xFFFFFFFFu;

	inline av_int64 make_handle(Kind kind, int device, uint32_t slot)
	{
		return (static_cast<av_int64>(kind) << 48) | (static_cast<av_int64>(device & 0xFFFF) << 32) | static_cast<av_int64>(slot);
	}
	inline bool handle_is(av_int64 h, Kind kind)
	{
		return h > 0 && ((h >> 48) & 0xFF) == kind;
	}
	inline int handle_device(av_int64 h)
	{
		return static_cast<int>((h >> 32) & 0xFFFF);
	}
	inline uint32_t handle_slot(av_int64 h)
	{
		return static_cast<uint32_t>(h & 0xFFFFFFFFll);
	}

	struct Context
	{
		int device = 0;
		hipStream_t stream = nullptr;
		bool is_default = false;
	};
	/* The byte ranges of an owning block written through the API, each with the number of its last write.  A write of a
	 * range that is already listed renews that entry (an arena that holds weights, activations and workspace sees the same few
	 * ranges over and over: every layer of a network writes one of two or three activation buffers), a new range takes the slot
	 * of the range written longest ago, and `lost` remembers the newest write whose range was dropped that way. */
	struct WriteLog
	{
		static constexpr int LOG = 64;
		std::mutex mutex;
		uint64_t version = 0; /* number of writes so far */
		uint64_t lost = 0; /* writes up to this number may have left the log */
		int used = 0;
		av_int64 lo[LOG], hi[LOG];
		uint64_t when[LOG];
		void record(av_int64 first, av_int64 last)
		{
			std::lock_guard<std::mutex> lock(mutex);
			version++;
			int oldest = 0;
			for (int i = 0; i < used; i++)
			{
				if (lo[i] == first && last == hi[i])
				{
					when[i] = version;
					return;
				}
				if (when[i] < when[oldest])
					oldest = i;
			}
			int slot = used;
			if (used < LOG)
				used++;
			else
			{
				slot = oldest;
				lost = std::max(lost, when[slot]);
			}
			lo[slot] = first;
			hi[slot] = last;
			when[slot] = version;
		}
		/* Whether bytes [first, last) were written after write number `seen`; `seen` moves up to the current number when not.
		 * Writes that have left the log count as hits. */
		bool written_since(uint64_t &seen, av_int64 first, av_int64 last)
		{
			std::lock_guard<std::mutex> lock(mutex);
			if (seen < lost)
				return true;
			for (int i = 0; i < used; i++)
				if (when[i] > seen && lo[i] < last && first < hi[i])
					return true;
			seen = version;
			return false;
		}
		uint64_t current()
		{
			std::lock_guard<std::mutex> lock(mutex);
			return version;
		}
	};
	struct Memory
	{
		char *data = nullptr;
		av_int64 size = 0;
		int device = 0;
		bool owning = true;
		uint32_t owner_slot = 0; /* for a view: slot of the owning block */
		uint64_t owner_uid = 0; /* for a view: uid of the owning block, so that a recycled slot is not mistaken for it */
		uint64_t uid = 0; /* unique over the life of the process */
		std::unique_ptr<WriteLog> writes; /* owning blocks only */
	};
	struct Tensor
	{
		avDataType_t dtype = AVOCADO_DTYPE_UNKNOWN;
		int nb_dims = 0;
		int dim[AVOCADO_MAX_TENSOR_DIMENSIONS] = { 0 };
		int dimension(int i) const
		{
			return (i >= 0 && i < nb_dims) ? dim[i] : 0;
		}
		int first_dim() const
		{
			return nb_dims > 0 ? dim[0] : 0;
		}
		int last_dim() const
		{
			return nb_dims > 0 ? dim[nb_dims - 1] : 0;
		}
		av_int64 volume() const
		{
			if (nb_dims == 0)
				return 0;
			av_int64 v = 1;
			for (int i = 0; i < nb_dims; i++)
				v *= dim[i];
			return v;
		}
		av_int64 volume_without_first_dim() const
		{
			if (nb_dims == 0)
				return 0;
			av_int64 v = 1;
			for (int i = 1; i < nb_dims; i++)
				v *= dim[i];
			return v;
		}
	};
	struct Convolution
	{
		avConvolutionMode_t mode = AVOCADO_CONVOLUTION_MODE;
		int nb_dims = 2;
		int padding[3] = { 0, 0, 0 };
		int strides[3] = { 1, 1, 1 };
		int dilation[3] = { 1, 1, 1 };
		int groups = 1;
		unsigned char padding_value[16] = { 0 };
		bool padding_value_is_zero() const
		{
			for (int i = 0; i < 16; i++)
				if (padding_value[i] != 0)
					return false;
			return true;
		}
	};

	/* Slot table with a free list.  Lookups return nullptr for foreign handles and for slots that are free; a stale handle whose
	 * slot was handed out again resolves to the new object (views guard against that with the owner's uid). */
	template<typename T>
	class Table
	{
			std::vector<std::unique_ptr<T>> m_slots;
			std::vector<uint32_t> m_free;
			mutable std::mutex m_mutex;
		public:
			uint32_t insert(std::unique_ptr<T> obj)
			{
				std::lock_guard<std::mutex> lock(m_mutex);
				if (!m_free.empty())
				{
					const uint32_t slot = m_free.back();
					m_free.pop_back();
					m_slots[slot] = std::move(obj);
					return slot;
				}
				m_slots.push_back(std::move(obj));
				return static_cast<uint32_t>(m_slots.size() - 1);
			}
			T* get(uint32_t slot) const
			{
				std::lock_guard<std::mutex> lock(m_mutex);
				return slot < m_slots.size() ? m_slots[slot].get() : nullptr;
			}
			std::unique_ptr<T> remove(uint32_t slot)
			{
				std::lock_guard<std::mutex> lock(m_mutex);
				if (slot >= m_slots.size() || !m_slots[slot])
					return nullptr;
				std::unique_ptr<T> out = std::move(m_slots[slot]);
				m_free.push_back(slot);
				return out;
			}
	};

	Table<Context>& contexts()
	{
		static Table<Context> t;
		return t;
	}
	Table<Memory>& memories()
	{
		static Table<Memory> t;
		return t;
	}
	Table<Tensor>& tensors()
	{
		static Table<Tensor> t;
		return t;
	}
	Table<Convolution>& convolutions()
	{
		static Table<Convolution> t;
		return t;
	}

	int device_count()
	{
		static const int count = []()
		{
			int n = 0;
			if (hipGetDeviceCount(&n) != hipSuccess)
			{
				(void) hipGetLastError();
				n = 0;
			}
			return n;
		}();
		return count;
	}

	/* Resolves a context handle; default contexts are materialised on the fly. */
	bool get_context(avContextDescriptor_t h, Context &out)
	{
		if (!handle_is(h, KIND_CONTEXT))
			return false;
		if (handle_slot(h) == DEFAULT_SLOT)
		{
			const int dev = handle_device(h);
			if (dev < 0 || dev >= device_count())
				return false;
			out.device = dev;
			out.stream = nullptr;
			out.is_default = true;
			return true;
		}
		const Context *c = contexts().get(handle_slot(h));
		if (c == nullptr)
			return false;
		out = *c;
		return true;
	}
	Memory* get_memory(avMemoryDescriptor_t h)
	{
		return handle_is(h, KIND_MEMORY) ? memories().get(handle_slot(h)) : nullptr;
	}
	const Tensor* get_tensor(avTensorDescriptor_t h)
	{
		return handle_is(h, KIND_TENSOR) ? tensors().get(handle_slot(h)) : nullptr;
	}
	Tensor* get_tensor_mut(avTensorDescriptor_t h)
	{
		return handle_is(h, KIND_TENSOR) ? tensors().get(handle_slot(h)) : nullptr;
	}
	Convolution* get_convolution(avConvolutionDescriptor_t h)
	{
		return handle_is(h, KIND_CONVOLUTION) ? convolutions().get(handle_slot(h)) : nullptr;
	}
	/* Device address behind a memory handle, nullptr for an absent (invalid) handle. */
	char* pointer_of(avMemoryDescriptor_t h)
	{
		Memory *m = get_memory(h);
		return m != nullptr ? m->data : nullptr;
	}
	/* The owning block behind a memory object; nullptr for a view whose owner has been destroyed (even if its slot is in use again). */
	Memory* owner_of(Memory *m)
	{
		if (m == nullptr || m->owning)
			return m;
		Memory *o = memories().get(m->owner_slot);
		return (o != nullptr && o->owning && o->uid == m->owner_uid) ? o : nullptr;
	}
	/* Records that `bytes` bytes from `offset` of the memory behind h are about to be written (bytes < 0: all of it). */
	void touch(avMemoryDescriptor_t h, av_int64 offset = 0, av_int64 bytes = -1)
	{
		Memory *m = get_memory(h);
		Memory *o = owner_of(m);
		if (o == nullptr || !o->writes || m->data == nullptr)
			return;
		const av_int64 first = (m->data - o->data) + offset;
		o->writes->record(first, first + (bytes < 0 ? m->size - offset : bytes));
	}

	avStatus_t from_hip(hipError_t err)
	{
		switch (err)
		{
			case hipSuccess:
				return AVOCADO_STATUS_SUCCESS;
			case hipErrorOutOfMemory:
				return AVOCADO_STATUS_ALLOC_FAILED;
			case hipErrorInsufficientDriver:
				return AVOCADO_STATUS_INSUFFICIENT_DRIVER;
			default:
				return AVOCADO_STATUS_EXECUTION_FAILED;
		}
	}
	/* Launch errors are read back without synchronising, as checkForErrors does (src/utilities.hpp:55-58). */
	avStatus_t from_launcher(int rc)
	{
		if (rc == 0)
			return from_hip(hipGetLastError());
		if (rc > 0)
			return from_hip(static_cast<hipError_t>(rc));
		switch (rc)
		{
			case AVHIP_NOT_SUPPORTED:
				return AVOCADO_STATUS_NOT_SUPPORTED;
			case AVHIP_UNSUPPORTED_DATATYPE:
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			case AVHIP_BAD_PARAM:
				return AVOCADO_STATUS_BAD_PARAM;
			default:
				return AVOCADO_STATUS_INTERNAL_ERROR;
		}
	}

	int size_of(avDataType_t dtype)
	{
		switch (dtype)
		{
			case AVOCADO_DTYPE_UINT8:
			case AVOCADO_DTYPE_INT8:
				return 1;
			case AVOCADO_DTYPE_INT16:
			case AVOCADO_DTYPE_FLOAT16:
			case AVOCADO_DTYPE_BFLOAT16:
				return 2;
			case AVOCADO_DTYPE_INT32:
			case AVOCADO_DTYPE_FLOAT32:
				return 4;
			case AVOCADO_DTYPE_INT64:
			case AVOCADO_DTYPE_FLOAT64:
			case AVOCADO_DTYPE_COMPLEX32:
				return 8;
			case AVOCADO_DTYPE_COMPLEX64:
				return 16;
			default:
				return 0;
		}
	}
	/* alpha / beta are host scalars: fp64 for fp64 tensors, fp32 otherwise (include/Avocado/cuda_backend.h:43-49). */
	double scalar_or(const void *p, avDataType_t tensor_dtype, double fallback)
	{
		if (p == nullptr)
			return fallback;
		if (tensor_dtype == AVOCADO_DTYPE_FLOAT64)
			return *static_cast<const double*>(p);
		return static_cast<double>(*static_cast<const float*>(p));
	}
	bool is_floating(avDataType_t t)
	{
		return t == AVOCADO_DTYPE_FLOAT16 || t == AVOCADO_DTYPE_BFLOAT16 || t == AVOCADO_DTYPE_FLOAT32 || t == AVOCADO_DTYPE_FLOAT64;
	}
	/* src/im2row.cu:75-81: every spatial extent of the filter equals `expected`. */
	bool is_conv(int expected, const Tensor &w)
	{
		for (int i = 0; i < w.nb_dims - 2; i++)
			if (w.dimension(1 + i) != expected)
				return false;
		return true;
	}
	bool fits(const Memory *m, av_int64 bytes)
	{
		return m != nullptr && m->data != nullptr && bytes <= m->size;
	}

	/* Everything the convolution entry points share: validated geometry in the launcher's POD form. */
	struct ConvProblem
	{
		avhipConvShape shape;
		avDataType_t x_dtype, w_dtype, y_dtype;
		const Convolution *conv;
	};
	avStatus_t make_problem(const Convolution *conv, const Tensor *x, const Tensor *w, const Tensor *y, ConvProblem &p)
	{
		if (conv == nullptr || x == nullptr || w == nullptr || y == nullptr)
			return AVOCADO_STATUS_BAD_PARAM;
		if (x->nb_dims != 4 || w->nb_dims != 4 || y->nb_dims != 4 || conv->nb_dims != 2)
			return AVOCADO_STATUS_NOT_SUPPORTED;
		if (conv->groups != 1)
			return AVOCADO_STATUS_NOT_SUPPORTED;
		if (x->dim[3] != w->dim[3] || y->dim[3] != w->dim[0] || x->dim[0] != y->dim[0])
			return AVOCADO_STATUS_BAD_PARAM;
		for (int i = 0; i < 4; i++)
			if (x->dim[i] <= 0 || w->dim[i] <= 0 || y->dim[i] <= 0)
				return AVOCADO_STATUS_BAD_PARAM;
		avhipConvShape &s = p.shape;
		s.N = x->dim[0];
		s.H = x->dim[1];
		s.W = x->dim[2];
		s.C = x->dim[3];
		s.K = w->dim[0];
		s.R = w->dim[1];
		s.S = w->dim[2];
		s.Ho = y->dim[1];
		s.Wo = y->dim[2];
		s.pad_h = conv->padding[0];
		s.pad_w = conv->padding[1];
		s.stride_h = conv->strides[0];
		s.stride_w = conv->strides[1];
		s.dil_h = conv->dilation[0];
		s.dil_w = conv->dilation[1];
		s.mode = (conv->mode == AVOCADO_CROSS_CORRELATION_MODE) ? 1 : 0;
		if (s.stride_h <= 0 || s.stride_w <= 0 || s.dil_h <= 0 || s.dil_w <= 0)
			return AVOCADO_STATUS_BAD_PARAM;
		/* The last window must start no later than one full (dilated) filter extent past the image: anything beyond would be
		 * an output made of padding only, which no caller means. */
		if (static_cast<av_int64>(s.Ho - 1) * s.stride_h + s.pad_h >= s.H || static_cast<av_int64>(s.Wo - 1) * s.stride_w + s.pad_w >= s.W)
			return AVOCADO_STATUS_BAD_PARAM;
		p.x_dtype = x->dtype;
		p.w_dtype = w->dtype;
		p.y_dtype = y->dtype;
		p.conv = conv;
		return AVOCADO_STATUS_SUCCESS;
	}

	/* ------------------------------------------------------------------------------------------------------------
	 * Cache of Winograd-transformed weights [t*t, K, C], keyed by the weight tensor (owning block, offset, shape, dtype, mode,
	 * tile size).  Rules that keep it safe with several contexts, rewritten weights and captured graphs:
	 *  - An entry records the event behind its transform and the stream that ran it.  A call on another stream waits for
	 *    that event (hipStreamWaitEvent) until the event is known to have completed.
	 *  - When the weight bytes were written through the API since the transform, the SAME buffer is transformed again on the
	 *    calling stream.  Whatever ordering the caller needs anyway between the write of the weights and other streams still
	 *    reading them also orders the rewrite of the matrices, and a captured graph that holds the buffer's address keeps
	 *    reading valid memory.  Nothing is freed on that path.
	 *  - Buffers are freed only by avhipInvalidateCaches, by the destruction of the weight block, or when the cache outgrows
	 *    its budget at the insertion of a new tensor, then after a synchronisation of the entry's device and outside the
	 *    cache's mutex.  The budget never takes an entry that a capturing stream was handed (a graph holds its address and may
	 *    be replayed at any time: such entries are pinned until avhipInvalidateCaches or the destruction of the weight block,
	 *    which are the two events that invalidate graphs) nor one that a caller was handed and has not yet enqueued its
	 *    kernel for (the lease returned with the matrices counts those; the device synchronisation only covers kernels that
	 *    are already enqueued).
	 *  - A stream that is capturing never changes the cache: no allocation, no transform, no event.  It may use an entry that
	 *    is up to date and whose transform ran on the same stream or is known to be complete; otherwise the lookup reports
	 *    AVOCADO_STATUS_BAD_ALLOC ("cannot allocate here": call once outside capture first) and the dispatcher takes the
	 *    implicit-GEMM plan, which needs no matrices.
	 * ------------------------------------------------------------------------------------------------------------ */
	struct WeightKey
	{
		uint64_t uid;
		av_int64 offset;
		int K, C, dtype, mode, m; /* m: Winograd output tile, 2 = F(2x2,3x3) for the fused kernel, 4 = F(4x4,3x3) for the non-fused plan,
		                           * 1 = F(2,3) along rows in the operand layout of the row-Winograd kernel, 3 = the weights themselves in the
		                           * operand layout of the stride-2 kernel (no transform) */
		bool operator<(const WeightKey &o) const
		{
			return std::tie(uid, offset, K, C, dtype, mode, m) < std::tie(o.uid, o.offset, o.K, o.C, o.dtype, o.mode, o.m);
		}
	};
	struct WeightEntry
	{
		void *U = nullptr;
		size_t bytes = 0;
		int device = 0;
		hipEvent_t ready = nullptr; /* recorded behind the last transform */
		hipStream_t stream = nullptr; /* the stream that ran it */
		bool complete = false; /* the event has been seen complete */
		uint64_t seen = 0; /* write number of the weight block the matrices are known to be current for */
		uint64_t last_use = 0;
		bool pinned = false; /* handed to a capturing stream: a graph holds the address */
		int in_use = 0; /* callers that hold the address and have not enqueued their kernel yet */
	};
	struct WeightCache
	{
		size_t budget = static_cast<size_t>(4) << 30; /* bytes of matrices kept before the least recently used go */
		std::mutex mutex;
		std::map<WeightKey, WeightEntry> entries;
		size_t total = 0;
		uint64_t clock = 0;
		uint64_t transforms = 0; /* weight transforms launched so far */
		static void release(std::vector<WeightEntry> &victims)
		{
			if (victims.empty())
				return;
			/* Kernels already enqueued on any stream of an entry's device may still read its matrices: that device is
			 * synchronised before the buffer goes.  Another thread may be capturing a stream in the global mode, under which
			 * a synchronisation or a free from any thread would break its capture: this thread says that it knows. */
			int previous_device = 0;
			(void) hipGetDevice(&previous_device);
			hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
			(void) hipThreadExchangeStreamCaptureMode(&mode);
			for (WeightEntry &e : victims)
			{
				if (e.U == nullptr)
					continue; /* (entries of the policy probe own nothing) */
				(void) hipSetDevice(e.device);
				(void) hipDeviceSynchronize();
				(void) hipFree(e.U);
				(void) hipEventDestroy(e.ready);
			}
			(void) hipSetDevice(previous_device);
			(void) hipThreadExchangeStreamCaptureMode(&mode);
			(void) hipGetLastError();
			victims.clear();
		}
		void clear()
		{
			std::vector<WeightEntry> victims;
			{
				std::lock_guard<std::mutex> lock(mutex);
				for (auto &e : entries)
					victims.push_back(e.second);
				entries.clear();
				total = 0;
			}
			release(victims);
		}
		void drop_block(uint64_t uid)
		{
			std::vector<WeightEntry> victims;
			{
				std::lock_guard<std::mutex> lock(mutex);
				for (auto it = entries.begin(); it != entries.end();)
					if (it->first.uid == uid)
					{
						victims.push_back(it->second);
						total -= it->second.bytes;
						it = entries.erase(it);
					}
					else
						++it;
			}
			release(victims);
		}
		/* with the mutex held: moves least recently used entries out until `incoming` more bytes fit the budget; entries that
		 * a graph or a caller still holds stay, whatever the budget says */
		void make_room(size_t incoming, std::vector<WeightEntry> &victims)
		{
			while (total + incoming > budget)
			{
				auto oldest = entries.end();
				for (auto it = entries.begin(); it != entries.end(); ++it)
					if (!it->second.pinned && it->second.in_use == 0 && (oldest == entries.end() || it->second.last_use < oldest->second.last_use))
						oldest = it;
				if (oldest == entries.end())
					break;
				victims.push_back(oldest->second);
				total -= oldest->second.bytes;
				entries.erase(oldest);
			}
		}
	};
	WeightCache& weight_cache()
	{
		static WeightCache c;
		return c;
	}
	uint64_t next_uid()
	{
		static std::atomic<uint64_t> uid { 0 };
		return ++uid;
	}
	bool is_capturing(hipStream_t stream)
	{
		if (stream == nullptr)
			return false; /* the null stream cannot be captured */
		hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
		if (hipStreamIsCapturing(stream, &status) != hipSuccess)
		{
			(void) hipGetLastError();
			return true; /* be careful: behave as under capture */
		}
		return status != hipStreamCaptureStatusNone;
	}

	/* Held by a caller from the lookup of transformed weights until its kernel is enqueued: keeps the budget from freeing the
	 * matrices in between. */
	struct WeightLease
	{
		WeightKey key;
		bool held = false;
		WeightLease() = default;
		WeightLease(const WeightLease&) = delete;
		WeightLease& operator=(const WeightLease&) = delete;
		void take(const WeightKey &k, WeightEntry &e)
		{
			key = k;
			held = true;
			e.in_use++;
		}
		~WeightLease()
		{
			if (!held)
				return;
			WeightCache &cache = weight_cache();
			std::lock_guard<std::mutex> lock(cache.mutex);
			auto it = cache.entries.find(key);
			if (it != cache.entries.end() && it->second.in_use > 0)
				it->second.in_use--;
		}
	};

	/* Returns the [t*t, K, C] Winograd weight matrices F(m x m, 3x3) of a weight tensor in `mat_dtype`, (re)transforming on the
	 * context's stream when the cache has none or the weight bytes were written since.  The caller keeps `lease` alive until
	 * the kernel that reads the matrices is enqueued. */
	avStatus_t cached_winograd_weights(const Context &ctx, const ConvProblem &p, avMemoryDescriptor_t wMem, int m, avDataType_t mat_dtype, const void **U,
			WeightLease &lease)
	{
		Memory *wm = get_memory(wMem);
		Memory *owner = owner_of(wm);
		if (wm == nullptr || owner == nullptr || !owner->writes)
			return AVOCADO_STATUS_BAD_PARAM;
		const av_int64 offset = wm->data - owner->data;
		const av_int64 w_bytes = static_cast<av_int64>(p.shape.K) * p.shape.R * p.shape.S * p.shape.C * size_of(p.w_dtype);
		const WeightKey key { owner->uid, offset, p.shape.K, p.shape.C, static_cast<int>(p.w_dtype), p.shape.mode, m };
		const int t = m + 2;
		const size_t bytes = m == 1 ? static_cast<size_t>(avhip_winograd_rows_weight_bytes(p.shape.K, p.shape.C))
				: m == 3 ? static_cast<size_t>(avhip_conv2d_strided_weight_bytes(p.shape.K, p.shape.C))
				: m == 5 ? static_cast<size_t>(avhip_conv2d_pointwise_block_weight_bytes(p.shape.K, p.shape.C))
				: static_cast<size_t>(t * t) * p.shape.K * p.shape.C * size_of(mat_dtype);
		WeightCache &cache = weight_cache();
		std::vector<WeightEntry> victims;
		avStatus_t status = AVOCADO_STATUS_SUCCESS;
		{
			std::lock_guard<std::mutex> lock(cache.mutex);
			auto it = cache.entries.find(key);
			const bool found = it != cache.entries.end();
			const bool current = found && !owner->writes->written_since(it->second.seen, offset, offset + w_bytes);
			if (current)
			{
				WeightEntry &e = it->second;
				e.last_use = ++cache.clock;
				U[0] = e.U;
				const bool capturing = !e.pinned && is_capturing(ctx.stream); /* (a pinned entry need not ask again) */
				if (e.complete || e.stream == ctx.stream)
				{
					/* stream order, or nothing left to wait for.  Under capture the graph keeps the address: pinned from now on */
					e.pinned = e.pinned || capturing;
					lease.take(key, e);
					return AVOCADO_STATUS_SUCCESS;
				}
				if (capturing || (e.pinned && is_capturing(ctx.stream)))
					return AVOCADO_STATUS_BAD_ALLOC; /* an event from outside must not enter the capture */
				if (hipEventQuery(e.ready) == hipSuccess)
				{
					e.complete = true;
					lease.take(key, e);
					return AVOCADO_STATUS_SUCCESS;
				}
				(void) hipGetLastError(); /* hipErrorNotReady is not an error here */
				const avStatus_t waiting = from_hip(hipStreamWaitEvent(ctx.stream, e.ready, 0));
				if (waiting == AVOCADO_STATUS_SUCCESS)
					lease.take(key, e);
				return waiting;
			}
			if (is_capturing(ctx.stream))
				return AVOCADO_STATUS_BAD_ALLOC;
			if (!found)
			{
				cache.make_room(bytes, victims);
				WeightEntry e;
				e.bytes = bytes;
				e.device = ctx.device;
				if (hipMalloc(&e.U, bytes) != hipSuccess)
				{
					(void) hipGetLastError();
					status = AVOCADO_STATUS_ALLOC_FAILED;
				}
				else if (hipEventCreateWithFlags(&e.ready, hipEventDisableTiming) != hipSuccess)
				{
					(void) hipGetLastError();
					(void) hipFree(e.U);
					status = AVOCADO_STATUS_ALLOC_FAILED;
				}
				else
				{
					it = cache.entries.emplace(key, e).first;
					cache.total += bytes;
				}
			}
			if (status == AVOCADO_STATUS_SUCCESS)
			{
				WeightEntry &e = it->second;
				/* the write number is read before the transform is enqueued: a write that slips in between is seen next time */
				e.seen = owner->writes->current();
				const int rc = m == 1 ? avhip_winograd_rows_weight_transform(ctx.stream, p.w_dtype, p.shape.mode, wm->data, e.U, p.shape.K, p.shape.C)
						: m == 3 ? avhip_conv2d_strided_weight_layout(ctx.stream, p.w_dtype, p.shape.mode, wm->data, e.U, p.shape.K, p.shape.C)
						: m == 5 ? avhip_conv2d_pointwise_block_weight_layout(ctx.stream, p.w_dtype, wm->data, e.U, p.shape.K, p.shape.C)
						: avhip_winograd_weight_transform(ctx.stream, p.w_dtype, mat_dtype, m, 3, p.shape.mode, wm->data, e.U, p.shape.K, p.shape.C);
				status = from_launcher(rc);
				cache.transforms++;
				if (status == AVOCADO_STATUS_SUCCESS)
					status = from_hip(hipEventRecord(e.ready, ctx.stream));
				if (status == AVOCADO_STATUS_SUCCESS)
				{
					e.stream = ctx.stream;
					e.complete = false;
					e.last_use = ++cache.clock;
					U[0] = e.U;
					lease.take(key, e);
				}
				else
				{
					/* the buffer holds nothing usable: drop the entry (freed below, outside the mutex) */
					victims.push_back(e);
					cache.total -= e.bytes;
					cache.entries.erase(it);
				}
			}
		}
		WeightCache::release(victims);
		return status;
	}
	/* [16, K, C] for the fused kernel: fp16 matrices for 16-bit tensors, fp32 for fp32 */
	avStatus_t fused_weights(const Context &ctx, const ConvProblem &p, avMemoryDescriptor_t wMem, const void **U, WeightLease &lease)
	{
		const avDataType_t mat_dtype = (p.w_dtype == AVOCADO_DTYPE_FLOAT32) ? AVOCADO_DTYPE_FLOAT32 : AVOCADO_DTYPE_FLOAT16;
		return cached_winograd_weights(ctx, p, wMem, 2, mat_dtype, U, lease);
	}

	bool winograd_supported(int r, int m)
	{
		return (r == 3 && (m == 2 || m == 4)) || (r == 5 && m == 2);
	}
	bool matrix_dtype_ok(avDataType_t tensor, avDataType_t matrix)
	{
		if (tensor == matrix)
			return is_floating(tensor);
		if (tensor == AVOCADO_DTYPE_FLOAT16)
			return matrix == AVOCADO_DTYPE_FLOAT32;
		if (tensor == AVOCADO_DTYPE_BFLOAT16)
			return matrix == AVOCADO_DTYPE_FLOAT16 || matrix == AVOCADO_DTYPE_FLOAT32;
		return false;
	}

	avStatus_t gemm_common(avContextDescriptor_t context, avGemmOperation_t aOp, avGemmOperation_t bOp, const void *alpha, const Tensor *a,
			avMemoryDescriptor_t aMem, const Tensor *b, avMemoryDescriptor_t bMem, const void *beta, const Tensor *c, avMemoryDescriptor_t cMem, bool batched)
	{
		Context ctx;
		if (!get_context(context, ctx))
			return AVOCADO_STATUS_BAD_PARAM;
		if (a == nullptr || b == nullptr || c == nullptr)
			return AVOCADO_STATUS_BAD_PARAM;
		const int nd = batched ? 3 : 2;
		if (a->nb_dims != nd || b->nb_dims != nd || c->nb_dims != nd)
			return AVOCADO_STATUS_BAD_PARAM;
		const int o = batched ? 1 : 0;
		const bool ta = (aOp == AVOCADO_GEMM_OPERATION_T), tb = (bOp == AVOCADO_GEMM_OPERATION_T);
		const int batch = batched ? a->dim[0] : 1;
		const int M = ta ? a->dim[o + 1] : a->dim[o];
		const int K = ta ? a->dim[o] : a->dim[o + 1];
		const int Kb = tb ? b->dim[o + 1] : b->dim[o];
		const int N = tb ? b->dim[o] : b->dim[o + 1];
		if (K != Kb || c->dim[o] != M || c->dim[o + 1] != N)
			return AVOCADO_STATUS_BAD_PARAM;
		if (batched && (b->dim[0] != batch || c->dim[0] != batch))
			return AVOCADO_STATUS_BAD_PARAM;
		if (a->dtype != b->dtype)
			return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
		const int lda = a->last_dim(), ldb = b->last_dim(), ldc = c->last_dim();
		double al = scalar_or(alpha, c->dtype, 1.0), be = scalar_or(beta, c->dtype, 0.0);
		if (c->dtype == AVOCADO_DTYPE_INT32)
		{
			/* src/gemm.cpp:42-53 */
			if (a->dtype != AVOCADO_DTYPE_INT8)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (lda % 4 != 0 || ldb % 4 != 0)
				return AVOCADO_STATUS_BAD_PARAM;
			const int ia = static_cast<int>(al), ib = static_cast<int>(be);
			if ((ia != 0 && ia != 1) || (ib != 0 && ib != 1))
				return AVOCADO_STATUS_BAD_PARAM;
			al = ia;
			be = ib;
		}
		Memory *am = get_memory(aMem), *bm = get_memory(bMem), *cm = get_memory(cMem);
		if (!fits(am, a->volume() * size_of(a->dtype)) || !fits(bm, b->volume() * size_of(b->dtype)) || !fits(cm, c->volume() * size_of(c->dtype)))
			return AVOCADO_STATUS_BAD_PARAM;
		if (hipSetDevice(ctx.device) != hipSuccess)
			return AVOCADO_STATUS_EXECUTION_FAILED;
		touch(cMem);
		const int rc = avhip_gemm_batched(ctx.stream, a->dtype, c->dtype, ta ? 1 : 0, tb ? 1 : 0, am->data, bm->data, cm->data, batch, M, N, K, lda, ldb, ldc,
				batched ? a->volume_without_first_dim() : 0, batched ? b->volume_without_first_dim() : 0, batched ? c->volume_without_first_dim() : 0, al,
				be);
		return from_launcher(rc);
	}

	/* Common front half of the two direct convolution entry points. */
	struct ConvCall
	{
		Context ctx;
		ConvProblem problem;
		Memory *x, *w, *y;
		char *bias, *z;
		avDataType_t bias_dtype;
		double alpha1, alpha2, beta;
	};
	avStatus_t prepare_conv(avContextDescriptor_t context, avConvolutionDescriptor_t config, const void *alpha1, avTensorDescriptor_t xDesc,
			avMemoryDescriptor_t xMem, avTensorDescriptor_t wDesc, avMemoryDescriptor_t wMem, avTensorDescriptor_t bDesc, avMemoryDescriptor_t bMem,
			const void *alpha2, avTensorDescriptor_t zDesc, avMemoryDescriptor_t zMem, const void *beta, avTensorDescriptor_t yDesc,
			avMemoryDescriptor_t yMem, ConvCall &call)
	{
		if (!get_context(context, call.ctx))
			return AVOCADO_STATUS_BAD_PARAM;
		const Tensor *x = get_tensor(xDesc), *w = get_tensor(wDesc), *y = get_tensor(yDesc);
		const avStatus_t st = make_problem(get_convolution(config), x, w, y, call.problem);
		if (st != AVOCADO_STATUS_SUCCESS)
			return st;
		if (x->dtype != w->dtype)
			return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
		call.x = get_memory(xMem);
		call.w = get_memory(wMem);
		call.y = get_memory(yMem);
		if (!fits(call.x, x->volume() * size_of(x->dtype)) || !fits(call.w, w->volume() * size_of(w->dtype))
				|| !fits(call.y, y->volume() * size_of(y->dtype)))
			return AVOCADO_STATUS_BAD_PARAM;
		call.bias = pointer_of(bMem);
		call.z = pointer_of(zMem);
		call.bias_dtype = AVOCADO_DTYPE_UNKNOWN;
		if (call.bias != nullptr)
		{
			const Tensor *b = get_tensor(bDesc);
			if (b == nullptr || b->volume() != w->dim[0] || !fits(get_memory(bMem), b->volume() * size_of(b->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
			call.bias_dtype = b->dtype;
		}
		if (call.z != nullptr)
		{
			const Tensor *z = get_tensor(zDesc);
			if (z == nullptr || z->volume() != y->volume() || z->dtype != y->dtype || !fits(get_memory(zMem), z->volume() * size_of(z->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
		}
		const avDataType_t scalar_type = (y->dtype == AVOCADO_DTYPE_FLOAT64) ? AVOCADO_DTYPE_FLOAT64 : AVOCADO_DTYPE_FLOAT32;
		call.alpha1 = scalar_or(alpha1, scalar_type, 1.0);
		call.alpha2 = scalar_or(alpha2, scalar_type, 1.0);
		call.beta = scalar_or(beta, scalar_type, 0.0);
		if (hipSetDevice(call.ctx.device) != hipSuccess)
			return AVOCADO_STATUS_EXECUTION_FAILED;
		return AVOCADO_STATUS_SUCCESS;
	}
	const void* padding_value_or_null(const Convolution *conv)
	{
		return conv->padding_value_is_zero() ? nullptr : conv->padding_value;
	}

	avStatus_t run_implicit_gemm(const ConvCall &c, avMemoryDescriptor_t yMem, avActivationType_t activation, const float *requant_scale)
	{
		const ConvProblem &p = c.problem;
		if (is_floating(p.x_dtype))
		{
			if (p.x_dtype == AVOCADO_DTYPE_FLOAT64)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (p.y_dtype != p.x_dtype)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (c.bias != nullptr && c.bias_dtype != AVOCADO_DTYPE_FLOAT32)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
		}
		else if (p.x_dtype != AVOCADO_DTYPE_INT8)
			return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
		touch(yMem);
		const int rc = avhip_conv2d_implicit_gemm(c.ctx.stream, p.x_dtype, p.y_dtype, c.bias_dtype, &p.shape, c.x->data, c.w->data, c.bias, c.z, c.y->data,
				padding_value_or_null(p.conv), c.alpha1, c.alpha2, c.beta, activation, requant_scale);
		return from_launcher(rc);
	}
	/* Layers with few output pixels and a long k: the k range split across workgroups, partial sums in the caller's
	 * workspace.  NOT_SUPPORTED (nothing launched) when the layer is not of that kind or the workspace does not take it. */
	int64_t split_k_bytes(const ConvProblem &p)
	{
		int64_t bytes = 0;
		if (p.y_dtype != p.x_dtype || avhip_conv2d_split_k_workspace(p.x_dtype, &p.shape, &bytes) != 0)
			return 0;
		return bytes;
	}
	avStatus_t run_split_k(const ConvCall &c, Memory *ws, avMemoryDescriptor_t workspaceMem, avMemoryDescriptor_t yMem, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		const int64_t bytes = split_k_bytes(p);
		if (bytes == 0 || ws == nullptr || ws->data == nullptr || ws->size < bytes || (c.bias != nullptr && c.bias_dtype != AVOCADO_DTYPE_FLOAT32))
			return AVOCADO_STATUS_NOT_SUPPORTED;
		const int rc = avhip_conv2d_implicit_gemm_split_k(c.ctx.stream, p.x_dtype, &p.shape, c.x->data, c.w->data, c.bias, c.z, c.y->data,
				padding_value_or_null(p.conv), c.alpha1, c.alpha2, c.beta, activation, ws->data, ws->size);
		if (rc == AVHIP_NOT_SUPPORTED)
			return AVOCADO_STATUS_NOT_SUPPORTED;
		touch(workspaceMem, 0, bytes);
		touch(yMem);
		return from_launcher(rc);
	}
	bool fused_winograd_applicable(const ConvProblem &p)
	{
		const avhipConvShape &s = p.shape;
		return s.R == 3 && s.S == 3 && s.stride_h == 1 && s.stride_w == 1 && s.dil_h == 1 && s.dil_w == 1 && p.y_dtype == p.x_dtype
				&& (p.x_dtype == AVOCADO_DTYPE_FLOAT16 || p.x_dtype == AVOCADO_DTYPE_BFLOAT16 || p.x_dtype == AVOCADO_DTYPE_FLOAT32)
				&& p.conv->padding_value_is_zero();
	}
	avStatus_t run_fused_winograd(const ConvCall &c, avMemoryDescriptor_t wMem, avMemoryDescriptor_t yMem, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		if (!fused_winograd_applicable(p))
			return AVOCADO_STATUS_NOT_SUPPORTED;
		if (c.bias != nullptr && c.bias_dtype != AVOCADO_DTYPE_FLOAT32)
			return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
		const void *U = nullptr;
		WeightLease lease;
		const avStatus_t st = fused_weights(c.ctx, p, wMem, &U, lease);
		if (st != AVOCADO_STATUS_SUCCESS)
			return st;
		touch(yMem);
		const int rc = avhip_conv2d_winograd_fused(c.ctx.stream, p.x_dtype, &p.shape, c.x->data, U, c.bias, c.z, c.y->data, c.alpha1, c.alpha2, c.beta,
				activation);
		return from_launcher(rc);
	}

	/* Row-wise Winograd F(2,3) for 16-bit 3x3 layers whose image bands fit a compute unit's LDS (conv_winograd_rows.hip): two
	 * thirds of the direct kernel's MFMA work.  Worth it when its workgroups (one per compute unit, 128 filters each) cover
	 * more than half of the chip and most of their 128 GEMM rows are image (15 x 15 images, 128 -> 128, bf16: 14.3 us against
	 * 13.2 us in the image-tile kernel at 128 images, 14.8 against 17.3 us at 160). */
	bool rows_winograd_pays(const ConvCall &c, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		if (p.y_dtype != p.x_dtype || !p.conv->padding_value_is_zero() || c.beta != 0.0 || (c.bias != nullptr && c.bias_dtype != AVOCADO_DTYPE_FLOAT32))
			return false;
		if (activation != AVOCADO_ACTIVATION_LINEAR && activation != AVOCADO_ACTIVATION_RELU)
			return false;
		int workgroups = 0, rows_used = 0;
		if (avhip_conv2d_winograd_rows_plan(p.x_dtype, &p.shape, &workgroups, &rows_used) != 0)
			return false;
		return avhip_set_winograd_rows(-1) == 2 || (workgroups >= 144 && rows_used >= 96);
	}
	avStatus_t run_rows_winograd(const ConvCall &c, avMemoryDescriptor_t wMem, avMemoryDescriptor_t yMem, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		const void *U = nullptr;
		WeightLease lease;
		const avStatus_t st = cached_winograd_weights(c.ctx, p, wMem, 1, AVOCADO_DTYPE_FLOAT16, &U, lease);
		if (st != AVOCADO_STATUS_SUCCESS)
			return st;
		const int rc = avhip_conv2d_winograd_rows(c.ctx.stream, p.x_dtype, &p.shape, c.x->data, U, c.bias, c.z, c.y->data, c.alpha1, c.alpha2, c.beta,
				activation);
		if (rc == AVHIP_NOT_SUPPORTED)
			return AVOCADO_STATUS_NOT_SUPPORTED;
		touch(yMem);
		return from_launcher(rc);
	}

	/* 3x3 stride-2 layers of 16-bit tensors through the parity-plane kernel (conv_strided.hip), weights in its operand layout from
	 * the cache.  Worth it from 96 workgroups (one per compute unit, 256 filters each) on: 56 x 56 x 128 -> 256 in bf16 takes 23.5
	 * us against 28.2 us in the gather kernel at 24 images (96 workgroups), 22.7 against 22.7 at 16. */
	bool strided_kernel_pays(const ConvCall &c, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		if (p.y_dtype != p.x_dtype || !p.conv->padding_value_is_zero() || c.beta != 0.0 || (c.bias != nullptr && c.bias_dtype != AVOCADO_DTYPE_FLOAT32))
			return false;
		if (activation != AVOCADO_ACTIVATION_LINEAR && activation != AVOCADO_ACTIVATION_RELU)
			return false;
		int workgroups = 0, rows_used = 0;
		if (avhip_conv2d_strided_plan(p.x_dtype, &p.shape, &workgroups, &rows_used) != 0)
			return false;
		return avhip_set_conv_strided(-1) == 2 || (workgroups >= 96 && rows_used >= 144);
	}
	avStatus_t run_strided_kernel(const ConvCall &c, avMemoryDescriptor_t wMem, avMemoryDescriptor_t yMem, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		const void *U = nullptr;
		WeightLease lease;
		const avStatus_t st = cached_winograd_weights(c.ctx, p, wMem, 3, p.w_dtype, &U, lease);
		if (st != AVOCADO_STATUS_SUCCESS)
			return st;
		const int rc = avhip_conv2d_strided(c.ctx.stream, p.x_dtype, &p.shape, c.x->data, U, c.bias, c.z, c.y->data, c.alpha1, c.alpha2, c.beta, activation);
		if (rc == AVHIP_NOT_SUPPORTED)
			return AVOCADO_STATUS_NOT_SUPPORTED;
		touch(yMem);
		return from_launcher(rc);
	}

	/* 1x1 layers of 16-bit tensors with 128 or 256 channels and a multiple of 512 filters through the pixel-block kernel
	 * (conv_pointwise_block.hip), weights in its operand layout from the cache (kind 5).  Worth it when its workgroups (one per
	 * compute unit) cover most of the chip with at least 96 pixels each: 28 x 28 x 256 -> 512 in bf16 takes 17.0 us against 18.0
	 * us in the short-k engine at 32 images (251 blocks of 100 pixels), 15.3 against 15.0 at 24. */
	bool pointwise_block_pays(const ConvCall &c, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		if (p.y_dtype != p.x_dtype || c.beta != 0.0 || (c.bias != nullptr && c.bias_dtype != AVOCADO_DTYPE_FLOAT32))
			return false;
		if (activation != AVOCADO_ACTIVATION_LINEAR && activation != AVOCADO_ACTIVATION_RELU)
			return false;
		int workgroups = 0, rows_used = 0;
		if (avhip_conv2d_pointwise_block_plan(p.x_dtype, &p.shape, &workgroups, &rows_used) != 0)
			return false;
		return avhip_set_pointwise_block(-1) == 2 || (workgroups >= 192 && rows_used >= 96);
	}
	avStatus_t run_pointwise_block(const ConvCall &c, avMemoryDescriptor_t wMem, avMemoryDescriptor_t yMem, avActivationType_t activation)
	{
		const ConvProblem &p = c.problem;
		const void *U = nullptr;
		WeightLease lease;
		const avStatus_t st = cached_winograd_weights(c.ctx, p, wMem, 5, p.w_dtype, &U, lease);
		if (st != AVOCADO_STATUS_SUCCESS)
			return st;
		const int rc = avhip_conv2d_pointwise_block(c.ctx.stream, p.x_dtype, &p.shape, c.x->data, U, c.bias, c.z, c.y->data, c.alpha1, c.alpha2, c.beta, activation);
		if (rc == AVHIP_NOT_SUPPORTED)
			return AVOCADO_STATUS_NOT_SUPPORTED;
		touch(yMem);
		return from_launcher(rc);
	}

	/* Non-fused Winograd F(4x4,3x3) through a caller workspace laid out as [V | M], each part 256-byte aligned; the transformed
	 * weights come from the library's cache (one transform per weight tensor and version). */
	struct NonFusedPlan
	{
		av_int64 v_bytes, m_bytes, total;
		int tiles;
		avDataType_t mat_dtype;
	};
	av_int64 align256(av_int64 v)
	{
		return (v + 255) / 256 * 256;
	}
	bool nonfused_plan(const ConvProblem &p, NonFusedPlan &plan)
	{
		const avhipConvShape &s = p.shape;
		if (!(s.R == 3 && s.S == 3 && s.stride_h == 1 && s.stride_w == 1 && s.dil_h == 1 && s.dil_w == 1 && p.x_dtype == AVOCADO_DTYPE_FLOAT32
				&& p.y_dtype == AVOCADO_DTYPE_FLOAT32 && s.Ho == s.H && s.Wo == s.W))
			return false;
		plan.mat_dtype = AVOCADO_DTYPE_FLOAT32;
		plan.tiles = s.N * ((s.H + 3) / 4) * ((s.W + 3) / 4);
		plan.v_bytes = align256(static_cast<av_int64>(36) * plan.tiles * s.C * 4);
		plan.m_bytes = align256(static_cast<av_int64>(36) * plan.tiles * s.K * 4);
		plan.total = plan.v_bytes + plan.m_bytes;
		return true;
	}
	/* Large fp32 layers: three HBM-bound passes around a batched GEMM that needs a quarter of the direct multiplications
	 * beat the fused kernel, which needs 4/9 of them and forms its operands in registers (measured on 256 x 15 x 15 x 128 ->
	 * 128: 16 + 56 + 18 us against 105 us; the weights are transformed once and cached).  Small ones do not fill the four launches. */
	bool nonfused_preferred(const ConvProblem &p, const NonFusedPlan &plan)
	{
		return plan.tiles >= 2048 && p.shape.C >= 64 && p.shape.K >= 64;
	}
	avStatus_t run_nonfused_winograd(const ConvCall &c, const NonFusedPlan &plan, Memory *ws, avMemoryDescriptor_t wMem, avMemoryDescriptor_t wsMem,
			avMemoryDescriptor_t yMem, avActivationType_t activation)
	{
		const avhipConvShape &s = c.problem.shape;
		char *V = ws->data, *Mx = V + plan.v_bytes;
		void *st = c.ctx.stream;
		const void *U = nullptr;
		WeightLease lease;
		const avStatus_t ws_status = cached_winograd_weights(c.ctx, c.problem, wMem, 4, plan.mat_dtype, &U, lease);
		if (ws_status != AVOCADO_STATUS_SUCCESS)
			return ws_status;
		touch(wsMem, 0, plan.total);
		int rc = avhip_winograd_input_transform(st, AVOCADO_DTYPE_FLOAT32, plan.mat_dtype, 4, 3, c.x->data, V, s.N, s.H, s.W, s.C, s.pad_h, s.pad_w,
					padding_value_or_null(c.problem.conv));
		if (rc == 0)
			rc = avhip_gemm_batched(st, plan.mat_dtype, plan.mat_dtype, 0, 1, V, U, Mx, 36, plan.tiles, s.K, s.C, s.C, s.C, s.K,
					static_cast<int64_t>(plan.tiles) * s.C, static_cast<int64_t>(s.K) * s.C, static_cast<int64_t>(plan.tiles) * s.K, 1.0, 0.0);
		if (rc == 0)
		{
			touch(yMem);
			rc = avhip_winograd_output_transform(st, AVOCADO_DTYPE_FLOAT32, plan.mat_dtype, 4, 3, Mx, c.y->data, c.bias, c.z, s.N, s.H, s.W, s.K, c.alpha1,
					c.alpha2, c.beta, activation);
		}
		return from_launcher(rc);
	}

	/* ------------------------------------------------------------------------------------------------------------
	 * Scratch of the one entry point that allocates nothing (avhipConvolutionWinogradFusedForwardNoAlloc): the transformed
	 * weights [16, K, C] of a call live in this fixed array instead of library-allocated memory.  Every device holds its
	 * own copy of the array at its own address until the process ends; the name below is a host-side stand-in, never a
	 * device address, so host code only ever uses the pointer that hipGetSymbolAddress returned for the current device.
	 * ------------------------------------------------------------------------------------------------------------ */
	static __device__ __align__(256) unsigned char scratch[AVHIP_NOALLOC_SCRATCH_BYTES];
	constexpr int NOALLOC_MAX_DEVICES = 64;
	/* Device address of `scratch` on `device`, which must be the current device.  Looked up once per device. */
	avStatus_t noalloc_scratch_pointer(int device, void **out)
	{
		static std::mutex mutex;
		static void *pointers[NOALLOC_MAX_DEVICES] = { nullptr };
		if (device < 0 || device >= NOALLOC_MAX_DEVICES)
			return AVOCADO_STATUS_BAD_PARAM;
		std::lock_guard<std::mutex> lock(mutex);
		if (pointers[device] == nullptr)
		{
			void *p = nullptr;
			const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
			if (err != hipSuccess || p == nullptr)
			{
				(void) hipGetLastError();
				return AVOCADO_STATUS_INTERNAL_ERROR;
			}
			pointers[device] = p;
		}
		out[0] = pointers[device];
		return AVOCADO_STATUS_SUCCESS;
	}

	/* Shared validation of the two per-channel transforms: the parameter tensors hold one value per element of x's
	 * trailing dimensions (volume(params) must divide volume(x)); fp32 parameters for 16-bit and fp32 tensors, fp64 for fp64. */
	avStatus_t per_channel_view(const Tensor *x, const Tensor *y, const Tensor *params, av_int64 &first, av_int64 &last)
	{
		if (x == nullptr || y == nullptr || params == nullptr || x->nb_dims == 0)
			return AVOCADO_STATUS_BAD_PARAM;
		if (!is_floating(x->dtype))
			return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
		if (x->dtype != y->dtype || x->volume() != y->volume())
			return AVOCADO_STATUS_BAD_PARAM;
		const avDataType_t param_type = (x->dtype == AVOCADO_DTYPE_FLOAT64) ? AVOCADO_DTYPE_FLOAT64 : AVOCADO_DTYPE_FLOAT32;
		if (params->dtype != param_type)
			return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
		last = params->volume();
		if (last <= 0 || x->volume() % last != 0)
			return AVOCADO_STATUS_BAD_PARAM;
		first = x->volume() / last;
		return AVOCADO_STATUS_SUCCESS;
	}
}

namespace avocado
{
	namespace backend
	{
		/* ---------------------------------------------------------------------------------------------------- device */
		int cudaGetNumberOfDevices()
		{
			return device_count();
		}
		avStatus_t cudaGetDeviceProperty(avDeviceIndex_t index, avDeviceProperty_t propertyName, void *result)
		{
			if (result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (index < 0 || index >= device_count())
				return AVOCADO_STATUS_BAD_PARAM;
			hipDeviceProp_t prop;
			if (hipGetDeviceProperties(&prop, index) != hipSuccess)
				return AVOCADO_STATUS_INTERNAL_ERROR;
			switch (propertyName)
			{
				case AVOCADO_DEVICE_NAME:
					std::memset(result, 0, 256);
					std::strncpy(static_cast<char*>(result), prop.name, 255);
					break;
				case AVOCADO_DEVICE_PROCESSOR_COUNT:
					static_cast<int32_t*>(result)[0] = prop.multiProcessorCount;
					break;
				case AVOCADO_DEVICE_MEMORY:
					static_cast<int64_t*>(result)[0] = static_cast<int64_t>(prop.totalGlobalMem);
					break;
				case AVOCADO_DEVICE_SUPPORTS_HALF_PRECISION:
				case AVOCADO_DEVICE_SUPPORTS_BFLOAT16:
				case AVOCADO_DEVICE_SUPPORTS_SINGLE_PRECISION:
				case AVOCADO_DEVICE_SUPPORTS_DOUBLE_PRECISION:
				case AVOCADO_DEVICE_SUPPORTS_DP4A: /* int8 dot products: MFMA i8 and v_dot4 */
				case AVOCADO_DEVICE_SUPPORTS_TENSOR_CORES: /* matrix cores */
					static_cast<bool*>(result)[0] = true;
					break;
				case AVOCADO_DEVICE_SUPPORTS_SSE:
				case AVOCADO_DEVICE_SUPPORTS_SSE2:
				case AVOCADO_DEVICE_SUPPORTS_SSE3:
				case AVOCADO_DEVICE_SUPPORTS_SSSE3:
				case AVOCADO_DEVICE_SUPPORTS_SSE41:
				case AVOCADO_DEVICE_SUPPORTS_SSE42:
				case AVOCADO_DEVICE_SUPPORTS_AVX:
				case AVOCADO_DEVICE_SUPPORTS_AVX2:
				case AVOCADO_DEVICE_SUPPORTS_AVX512_F:
				case AVOCADO_DEVICE_SUPPORTS_AVX512_VL_BW_DQ:
					static_cast<bool*>(result)[0] = false;
					break;
				case AVOCADO_DEVICE_ARCH_MAJOR:
					static_cast<int32_t*>(result)[0] = prop.major;
					break;
				case AVOCADO_DEVICE_ARCH_MINOR:
					static_cast<int32_t*>(result)[0] = prop.minor;
					break;
				default:
					return AVOCADO_STATUS_BAD_PARAM;
			}
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaIsCopyPossible(avDeviceIndex_t from, avDeviceIndex_t to, bool *result)
		{
			if (result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			result[0] = (from == to);
			return AVOCADO_STATUS_SUCCESS;
		}

		/* --------------------------------------------------------------------------------------------------- context */
		avStatus_t cudaCreateContextDescriptor(avContextDescriptor_t *result, avDeviceIndex_t deviceIndex)
		{
			if (result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (deviceIndex < 0 || deviceIndex >= device_count())
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(deviceIndex) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			std::unique_ptr<Context> ctx(new Context());
			ctx->device = deviceIndex;
			if (hipStreamCreate(&ctx->stream) != hipSuccess) /* default priority; ordered against the null stream */
				return AVOCADO_STATUS_BAD_ALLOC;
			result[0] = make_handle(KIND_CONTEXT, deviceIndex, contexts().insert(std::move(ctx)));
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaDestroyContextDescriptor(avContextDescriptor_t desc)
		{
			if (!handle_is(desc, KIND_CONTEXT) || handle_slot(desc) == DEFAULT_SLOT)
				return AVOCADO_STATUS_BAD_PARAM;
			std::unique_ptr<Context> ctx = contexts().remove(handle_slot(desc));
			if (!ctx)
				return AVOCADO_STATUS_BAD_PARAM;
			(void) hipSetDevice(ctx->device);
			if (hipStreamDestroy(ctx->stream) != hipSuccess)
				return AVOCADO_STATUS_FREE_FAILED;
			return AVOCADO_STATUS_SUCCESS;
		}
		avContextDescriptor_t cudaGetDefaultContext(avDeviceIndex_t deviceIndex)
		{
			if (deviceIndex >= 0 && deviceIndex < device_count())
				return make_handle(KIND_CONTEXT, deviceIndex, DEFAULT_SLOT);
			return static_cast<avContextDescriptor_t>(-1);
		}
		avStatus_t cudaSynchronizeWithContext(avContextDescriptor_t context)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess || hipStreamSynchronize(ctx.stream) != hipSuccess)
				return AVOCADO_STATUS_INTERNAL_ERROR;
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaIsContextReady(avContextDescriptor_t context, bool *result)
		{
			if (result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			(void) hipSetDevice(ctx.device);
			const hipError_t st = hipStreamQuery(ctx.stream);
			result[0] = (st == hipSuccess);
			if (st == hipSuccess || st == hipErrorNotReady)
				return AVOCADO_STATUS_SUCCESS;
			return from_hip(st);
		}

		/* ---------------------------------------------------------------------------------------------------- memory */
		avStatus_t cudaCreateMemoryDescriptor(avMemoryDescriptor_t *result, avDeviceIndex_t deviceIndex, av_int64 sizeInBytes)
		{
			if (result == nullptr || sizeInBytes < 0)
				return AVOCADO_STATUS_BAD_PARAM;
			if (deviceIndex < 0 || deviceIndex >= device_count())
				return AVOCADO_STATUS_BAD_PARAM;
			std::unique_ptr<Memory> m(new Memory());
			m->device = deviceIndex;
			m->size = sizeInBytes;
			m->owning = true;
			m->uid = next_uid();
			m->writes.reset(new WriteLog());
			if (sizeInBytes > 0)
			{
				if (hipSetDevice(deviceIndex) != hipSuccess)
					return AVOCADO_STATUS_EXECUTION_FAILED;
				void *p = nullptr;
				if (hipMalloc(&p, static_cast<size_t>(sizeInBytes)) != hipSuccess)
				{
					(void) hipGetLastError();
					return AVOCADO_STATUS_BAD_ALLOC;
				}
				m->data = static_cast<char*>(p);
			}
			result[0] = make_handle(KIND_MEMORY, deviceIndex, memories().insert(std::move(m)));
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaCreateMemoryView(avMemoryDescriptor_t *result, const avMemoryDescriptor_t desc, av_int64 sizeInBytes, av_int64 offsetInBytes)
		{
			if (result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *src = get_memory(desc);
			if (src == nullptr || !src->owning || offsetInBytes < 0 || sizeInBytes < 0 || offsetInBytes + sizeInBytes > src->size)
				return AVOCADO_STATUS_BAD_PARAM;
			std::unique_ptr<Memory> m(new Memory());
			m->device = src->device;
			m->size = sizeInBytes;
			m->owning = false;
			m->owner_slot = handle_slot(desc);
			m->owner_uid = src->uid;
			m->data = src->data != nullptr ? src->data + offsetInBytes : nullptr;
			m->uid = next_uid();
			result[0] = make_handle(KIND_MEMORY, src->device, memories().insert(std::move(m)));
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaDestroyMemoryDescriptor(avMemoryDescriptor_t desc)
		{
			if (!handle_is(desc, KIND_MEMORY))
				return AVOCADO_STATUS_BAD_PARAM;
			std::unique_ptr<Memory> m = memories().remove(handle_slot(desc));
			if (!m)
				return AVOCADO_STATUS_BAD_PARAM;
			if (m->owning)
			{
				weight_cache().drop_block(m->uid);
				if (m->data != nullptr)
				{
					(void) hipSetDevice(m->device);
					if (hipFree(m->data) != hipSuccess)
						return AVOCADO_STATUS_FREE_FAILED;
				}
			}
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaSetMemory(avContextDescriptor_t context, avMemoryDescriptor_t dst, av_int64 dstOffset, av_int64 dstSize, const void *pattern,
				av_int64 patternSize)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *m = get_memory(dst);
			if (m == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (m->data == nullptr)
				return dstSize != 0 ? AVOCADO_STATUS_BAD_PARAM : AVOCADO_STATUS_SUCCESS;
			if (dstOffset < 0 || dstSize < 0 || dstOffset + dstSize > m->size)
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			if (dstSize == 0)
				return AVOCADO_STATUS_SUCCESS;
			touch(dst, dstOffset, dstSize);
			avStatus_t st;
			if (pattern == nullptr)
			{
				/* a fill kernel rather than a memset node, so that the call stays safe under stream capture */
				static const unsigned char zeros[16] = { 0 };
				int width = 16;
				while (width > 1 && (dstSize % width != 0 || reinterpret_cast<uintptr_t>(m->data + dstOffset) % width != 0))
					width /= 2;
				st = from_launcher(avhip_set_memory(ctx.stream, m->data + dstOffset, dstSize, zeros, width));
			}
			else
			{
				if (patternSize != 1 && patternSize != 2 && patternSize != 4 && patternSize != 8 && patternSize != 16)
					return AVOCADO_STATUS_BAD_PARAM;
				if (dstSize % patternSize != 0 || dstOffset % patternSize != 0)
					return AVOCADO_STATUS_BAD_PARAM;
				st = from_launcher(avhip_set_memory(ctx.stream, m->data + dstOffset, dstSize, pattern, static_cast<int>(patternSize)));
			}
			/* the default context is synchronous (src/descriptors.cu:78-80 of the reference) */
			if (st == AVOCADO_STATUS_SUCCESS && ctx.is_default)
				return from_hip(hipStreamSynchronize(ctx.stream));
			return st;
		}
		avStatus_t cudaCopyMemory(avContextDescriptor_t context, avMemoryDescriptor_t dst, av_int64 dstOffset, const avMemoryDescriptor_t src,
				av_int64 srcOffset, av_int64 count)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *d = get_memory(dst), *s = get_memory(src);
			if (d == nullptr || s == nullptr || count < 0 || dstOffset < 0 || srcOffset < 0 || dstOffset + count > d->size || srcOffset + count > s->size)
				return AVOCADO_STATUS_BAD_PARAM;
			if (count == 0)
				return AVOCADO_STATUS_SUCCESS;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(dst, dstOffset, count);
			if (ctx.is_default)
				return from_hip(hipMemcpy(d->data + dstOffset, s->data + srcOffset, static_cast<size_t>(count), hipMemcpyDeviceToDevice));
			return from_hip(hipMemcpyAsync(d->data + dstOffset, s->data + srcOffset, static_cast<size_t>(count), hipMemcpyDeviceToDevice, ctx.stream));
		}
		avStatus_t cudaCopyMemoryToHost(avContextDescriptor_t context, void *dst, const avMemoryDescriptor_t src, av_int64 srcOffset, av_int64 bytes)
		{
			if (dst == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *s = get_memory(src);
			if (s == nullptr || bytes < 0 || srcOffset < 0 || srcOffset + bytes > s->size)
				return AVOCADO_STATUS_BAD_PARAM;
			if (bytes == 0)
				return AVOCADO_STATUS_SUCCESS;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			if (ctx.is_default)
				return from_hip(hipMemcpy(dst, s->data + srcOffset, static_cast<size_t>(bytes), hipMemcpyDeviceToHost));
			return from_hip(hipMemcpyAsync(dst, s->data + srcOffset, static_cast<size_t>(bytes), hipMemcpyDeviceToHost, ctx.stream));
		}
		avStatus_t cudaCopyMemoryFromHost(avContextDescriptor_t context, avMemoryDescriptor_t dst, av_int64 dstOffset, const void *src, av_int64 bytes)
		{
			if (src == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *d = get_memory(dst);
			if (d == nullptr || bytes < 0 || dstOffset < 0 || dstOffset + bytes > d->size)
				return AVOCADO_STATUS_BAD_PARAM;
			if (bytes == 0)
				return AVOCADO_STATUS_SUCCESS;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(dst, dstOffset, bytes);
			if (ctx.is_default)
				return from_hip(hipMemcpy(d->data + dstOffset, src, static_cast<size_t>(bytes), hipMemcpyHostToDevice));
			return from_hip(hipMemcpyAsync(d->data + dstOffset, src, static_cast<size_t>(bytes), hipMemcpyHostToDevice, ctx.stream));
		}
		avStatus_t cudaPageLock(void *ptr, av_int64 count)
		{
			(void) count;
			if (ptr == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			return AVOCADO_STATUS_NOT_SUPPORTED;
		}
		avStatus_t cudaPageUnlock(void *ptr)
		{
			if (ptr == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			return AVOCADO_STATUS_NOT_SUPPORTED;
		}

		/* ----------------------------------------------------------------------------------------- tensor descriptor */
		avStatus_t cudaCreateTensorDescriptor(avTensorDescriptor_t *result)
		{
			if (result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			result[0] = make_handle(KIND_TENSOR, 0, tensors().insert(std::unique_ptr<Tensor>(new Tensor())));
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaDestroyTensorDescriptor(avTensorDescriptor_t desc)
		{
			if (!handle_is(desc, KIND_TENSOR) || !tensors().remove(handle_slot(desc)))
				return AVOCADO_STATUS_BAD_PARAM;
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaSetTensorDescriptor(avTensorDescriptor_t desc, avDataType_t dtype, int nbDims, const int dimensions[])
		{
			if (nbDims < 0 || nbDims > AVOCADO_MAX_TENSOR_DIMENSIONS)
				return AVOCADO_STATUS_BAD_PARAM;
			if (dimensions == nullptr && nbDims != 0)
				return AVOCADO_STATUS_BAD_PARAM;
			Tensor *t = get_tensor_mut(desc);
			if (t == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			t->dtype = dtype;
			t->nb_dims = nbDims;
			for (int i = 0; i < AVOCADO_MAX_TENSOR_DIMENSIONS; i++)
				t->dim[i] = i < nbDims ? dimensions[i] : 0;
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaGetTensorDescriptor(avTensorDescriptor_t desc, avDataType_t *dtype, int *nbDims, int dimensions[])
		{
			const Tensor *t = get_tensor(desc);
			if (t == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (dtype != nullptr)
				dtype[0] = t->dtype;
			if (nbDims != nullptr)
				nbDims[0] = t->nb_dims;
			if (dimensions != nullptr)
				for (int i = 0; i < t->nb_dims; i++)
					dimensions[i] = t->dim[i];
			return AVOCADO_STATUS_SUCCESS;
		}

		/* ------------------------------------------------------------------------------------ convolution descriptor */
		avStatus_t cudaCreateConvolutionDescriptor(avConvolutionDescriptor_t *result)
		{
			if (result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			result[0] = make_handle(KIND_CONVOLUTION, 0, convolutions().insert(std::unique_ptr<Convolution>(new Convolution())));
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaDestroyConvolutionDescriptor(avConvolutionDescriptor_t desc)
		{
			if (!handle_is(desc, KIND_CONVOLUTION) || !convolutions().remove(handle_slot(desc)))
				return AVOCADO_STATUS_BAD_PARAM;
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaSetConvolutionDescriptor(avConvolutionDescriptor_t desc, avConvolutionMode_t mode, int nbDims, const int padding[],
				const int strides[], const int dilation[], int groups, const void *paddingValue)
		{
			Convolution *c = get_convolution(desc);
			if (c == nullptr || nbDims < 1 || nbDims > 3 || groups <= 0)
				return AVOCADO_STATUS_BAD_PARAM;
			if (mode != AVOCADO_CONVOLUTION_MODE && mode != AVOCADO_CROSS_CORRELATION_MODE)
				return AVOCADO_STATUS_BAD_PARAM;
			c->mode = mode;
			c->nb_dims = nbDims;
			c->groups = groups;
			for (int i = 0; i < 3; i++)
			{
				c->padding[i] = (padding != nullptr && i < nbDims) ? padding[i] : 0;
				c->strides[i] = (strides != nullptr && i < nbDims) ? strides[i] : 1;
				c->dilation[i] = (dilation != nullptr && i < nbDims) ? dilation[i] : 1;
			}
			if (paddingValue != nullptr)
				std::memcpy(c->padding_value, paddingValue, 16);
			else
				std::memset(c->padding_value, 0, 16);
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t cudaGetConvolutionDescriptor(avConvolutionDescriptor_t desc, avConvolutionMode_t *mode, int *nbDims, int padding[], int strides[],
				int dilation[], int *groups, void *paddingValue)
		{
			const Convolution *c = get_convolution(desc);
			if (c == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (mode != nullptr)
				mode[0] = c->mode;
			if (nbDims != nullptr)
				nbDims[0] = c->nb_dims;
			if (groups != nullptr)
				groups[0] = c->groups;
			for (int i = 0; i < c->nb_dims; i++)
			{
				if (padding != nullptr)
					padding[i] = c->padding[i];
				if (strides != nullptr)
					strides[i] = c->strides[i];
				if (dilation != nullptr)
					dilation[i] = c->dilation[i];
			}
			if (paddingValue != nullptr)
				std::memcpy(paddingValue, c->padding_value, 16);
			return AVOCADO_STATUS_SUCCESS;
		}

		/* ----------------------------------------------------------------------------------------- tensor operations */
		avStatus_t cudaChangeType(avContextDescriptor_t context, avMemoryDescriptor_t dst, avDataType_t dstType, const avMemoryDescriptor_t src,
				avDataType_t srcType, av_int64 elements)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			if (elements < 0)
				return AVOCADO_STATUS_BAD_PARAM;
			if (size_of(dstType) == 0 || size_of(srcType) == 0)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			Memory *d = get_memory(dst), *s = get_memory(src);
			if (elements > 0 && (!fits(d, elements * size_of(dstType)) || !fits(s, elements * size_of(srcType))))
				return AVOCADO_STATUS_BAD_PARAM;
			if (elements == 0)
				return AVOCADO_STATUS_SUCCESS;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(dst, 0, elements * size_of(dstType));
			return from_launcher(avhip_change_type(ctx.stream, d->data, dstType, s->data, srcType, elements));
		}

		avStatus_t cudaAddBias(avContextDescriptor_t context, const void *alpha1, const void *alpha2, const avTensorDescriptor_t xDesc,
				const avMemoryDescriptor_t xMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const avTensorDescriptor_t yDesc,
				avMemoryDescriptor_t yMem, const void *beta1, const void *beta2, const void *beta3, const avMemoryDescriptor_t zMem,
				avActivationType_t activation)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Tensor *x = get_tensor(xDesc), *b = get_tensor(bDesc), *y = get_tensor(yDesc);
			if (x == nullptr || b == nullptr || y == nullptr || x->nb_dims == 0)
				return AVOCADO_STATUS_BAD_PARAM;
			if (!is_floating(y->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (x->dtype != y->dtype || x->volume() != y->volume())
				return AVOCADO_STATUS_BAD_PARAM;
			const avDataType_t bias_type = (y->dtype == AVOCADO_DTYPE_FLOAT64) ? AVOCADO_DTYPE_FLOAT64 : AVOCADO_DTYPE_FLOAT32;
			if (b->dtype != bias_type)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			const int last = x->last_dim();
			if (b->volume() != last || last <= 0)
				return AVOCADO_STATUS_BAD_PARAM;
			const av_int64 first = x->volume() / last;
			Memory *xm = get_memory(xMem), *bm = get_memory(bMem), *ym = get_memory(yMem);
			const av_int64 bytes = x->volume() * size_of(x->dtype);
			if (!fits(xm, bytes) || !fits(ym, bytes) || !fits(bm, static_cast<av_int64>(last) * size_of(bias_type)))
				return AVOCADO_STATUS_BAD_PARAM;
			const double a1 = scalar_or(alpha1, y->dtype, 1.0), a2 = scalar_or(alpha2, y->dtype, 1.0);
			const double b1 = scalar_or(beta1, y->dtype, 0.0), b2 = scalar_or(beta2, y->dtype, 0.0), b3 = scalar_or(beta3, y->dtype, 0.0);
			char *z = pointer_of(zMem);
			if ((b1 != 0.0 || b2 != 0.0) && !fits(get_memory(zMem), bytes))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(yMem);
			return from_launcher(avhip_add_bias(ctx.stream, y->dtype, xm->data, bm->data, z, ym->data, first, last, a1, a2, b1, b2, b3, activation));
		}

		avStatus_t cudaAffineForward(avContextDescriptor_t context, avActivationType_t activation, const avTensorDescriptor_t wDesc,
				const avMemoryDescriptor_t wMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha,
				const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const void *beta, const avTensorDescriptor_t yDesc,
				avMemoryDescriptor_t yMem)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Tensor *x = get_tensor(xDesc), *y = get_tensor(yDesc), *w = get_tensor(wDesc), *b = get_tensor(bDesc);
			av_int64 first = 0, last = 0;
			const avStatus_t st = per_channel_view(x, y, b, first, last);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			if (w == nullptr || w->dtype != b->dtype || w->volume() != last)
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *xm = get_memory(xMem), *ym = get_memory(yMem), *wm = get_memory(wMem), *bm = get_memory(bMem);
			const av_int64 bytes = x->volume() * size_of(x->dtype), param_bytes = last * size_of(b->dtype);
			if (!fits(xm, bytes) || !fits(ym, bytes) || !fits(wm, param_bytes) || !fits(bm, param_bytes))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(yMem);
			return from_launcher(avhip_affine_forward(ctx.stream, x->dtype, xm->data, ym->data, wm->data, bm->data, first, last,
					scalar_or(alpha, x->dtype, 1.0), scalar_or(beta, x->dtype, 0.0), activation));
		}

		avStatus_t cudaBatchNormInference(avContextDescriptor_t context, avActivationType_t activation, const void *alpha, const avTensorDescriptor_t xDesc,
				const avMemoryDescriptor_t xMem, const void *beta, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem,
				const avTensorDescriptor_t scaleBiasMeanVarDesc, const avMemoryDescriptor_t scaleMem, const avMemoryDescriptor_t biasMem,
				const avMemoryDescriptor_t meanMem, const avMemoryDescriptor_t varianceMem, double epsilon)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Tensor *x = get_tensor(xDesc), *y = get_tensor(yDesc), *params = get_tensor(scaleBiasMeanVarDesc);
			av_int64 first = 0, last = 0;
			const avStatus_t st = per_channel_view(x, y, params, first, last);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			if (!(epsilon >= 0.0))
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *xm = get_memory(xMem), *ym = get_memory(yMem);
			Memory *pm[4] = { get_memory(scaleMem), get_memory(biasMem), get_memory(meanMem), get_memory(varianceMem) };
			const av_int64 bytes = x->volume() * size_of(x->dtype), param_bytes = last * size_of(params->dtype);
			if (!fits(xm, bytes) || !fits(ym, bytes))
				return AVOCADO_STATUS_BAD_PARAM;
			for (int i = 0; i < 4; i++)
				if (!fits(pm[i], param_bytes))
					return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(yMem);
			return from_launcher(avhip_batchnorm_inference(ctx.stream, x->dtype, xm->data, ym->data, pm[0]->data, pm[1]->data, pm[2]->data, pm[3]->data,
					first, last, scalar_or(alpha, x->dtype, 1.0), scalar_or(beta, x->dtype, 0.0), epsilon, activation));
		}

		avStatus_t cudaGemm(avContextDescriptor_t context, avGemmOperation_t aOp, avGemmOperation_t bOp, const void *alpha,
				const avTensorDescriptor_t aDesc, const avMemoryDescriptor_t aMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem,
				const void *beta, const avTensorDescriptor_t cDesc, avMemoryDescriptor_t cMem)
		{
			return gemm_common(context, aOp, bOp, alpha, get_tensor(aDesc), aMem, get_tensor(bDesc), bMem, beta, get_tensor(cDesc), cMem, false);
		}
		avStatus_t cudaGemmBatched(avContextDescriptor_t context, avGemmOperation_t aOp, avGemmOperation_t bOp, const void *alpha,
				const avTensorDescriptor_t aDesc, const avMemoryDescriptor_t aMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem,
				const void *beta, const avTensorDescriptor_t cDesc, avMemoryDescriptor_t cMem)
		{
			return gemm_common(context, aOp, bOp, alpha, get_tensor(aDesc), aMem, get_tensor(bDesc), bMem, beta, get_tensor(cDesc), cMem, true);
		}

		/* ----------------------------------------------------------------------------------------------- convolution */
		avStatus_t cudaIm2Row(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const avTensorDescriptor_t filterDesc,
				const avTensorDescriptor_t srcDesc, const avMemoryDescriptor_t srcMem, const avTensorDescriptor_t rowDesc, avMemoryDescriptor_t rowMem)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Convolution *conv = get_convolution(config);
			const Tensor *f = get_tensor(filterDesc), *src = get_tensor(srcDesc), *row = get_tensor(rowDesc);
			if (conv == nullptr || f == nullptr || src == nullptr || row == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (f->nb_dims != 4 || src->nb_dims != 4 || row->nb_dims != 2 || conv->nb_dims != 2 || conv->groups != 1)
				return AVOCADO_STATUS_NOT_SUPPORTED;
			avhipConvShape s;
			s.N = src->dim[0];
			s.H = src->dim[1];
			s.W = src->dim[2];
			s.C = src->dim[3];
			s.K = f->dim[0];
			s.R = f->dim[1];
			s.S = f->dim[2];
			s.pad_h = conv->padding[0];
			s.pad_w = conv->padding[1];
			s.stride_h = conv->strides[0];
			s.stride_w = conv->strides[1];
			s.dil_h = conv->dilation[0];
			s.dil_w = conv->dilation[1];
			s.mode = (conv->mode == AVOCADO_CROSS_CORRELATION_MODE) ? 1 : 0;
			/* output extent of a convolution whose offset padding is mirrored at the far edge; strides and dilations are
			 * honoured (the reference's kernel, src/im2row.cu:29-66, is stride 1 only) */
			if (s.stride_h < 1 || s.stride_w < 1 || s.dil_h < 1 || s.dil_w < 1)
				return AVOCADO_STATUS_BAD_PARAM;
			const int span_h = s.H - 2 * s.pad_h - (s.dil_h * (s.R - 1) + 1), span_w = s.W - 2 * s.pad_w - (s.dil_w * (s.S - 1) + 1);
			if (span_h < 0 || span_w < 0)
				return AVOCADO_STATUS_BAD_PARAM;
			s.Ho = span_h / s.stride_h + 1;
			s.Wo = span_w / s.stride_w + 1;
			if (s.C != f->dim[3] || s.Ho <= 0 || s.Wo <= 0)
				return AVOCADO_STATUS_BAD_PARAM;
			if (row->dim[0] != static_cast<av_int64>(s.N) * s.Ho * s.Wo || row->dim[1] != s.R * s.S * s.C || row->dtype != src->dtype)
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *sm = get_memory(srcMem), *rm = get_memory(rowMem);
			if (!fits(sm, src->volume() * size_of(src->dtype)) || !fits(rm, row->volume() * size_of(row->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(rowMem);
			return from_launcher(avhip_im2row(ctx.stream, size_of(src->dtype), &s, sm->data, rm->data, padding_value_or_null(conv)));
		}

		avStatus_t cudaConvolutionImplicitGemmForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const void *alpha1,
				const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem,
				const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2, const avTensorDescriptor_t zDesc,
				const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem,
				avActivationType_t activation)
		{
			ConvCall call;
			const avStatus_t st = prepare_conv(context, config, alpha1, xDesc, xMem, wDesc, wMem, bDesc, bMem, alpha2, zDesc, zMem, beta, yDesc, yMem, call);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			/* the two implicit-GEMM kernels that want the weights in their own layout (stride 2; 1x1 with many filters): the same
			 * arithmetic, taken where they pay and the library's cache can hold the layout (not while the stream is capturing
			 * with a cold cache: nothing was launched then and the general kernels take over) */
			if (strided_kernel_pays(call, activation))
			{
				const avStatus_t rs = run_strided_kernel(call, wMem, yMem, activation);
				if (rs != AVOCADO_STATUS_NOT_SUPPORTED && rs != AVOCADO_STATUS_BAD_ALLOC)
					return rs;
			}
			if (pointwise_block_pays(call, activation))
			{
				const avStatus_t rs = run_pointwise_block(call, wMem, yMem, activation);
				if (rs != AVOCADO_STATUS_NOT_SUPPORTED && rs != AVOCADO_STATUS_BAD_ALLOC)
					return rs;
			}
			return run_implicit_gemm(call, yMem, activation, nullptr);
		}

		avStatus_t cudaConvolutionWinogradFusedForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const void *alpha1,
				const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem,
				const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2, const avTensorDescriptor_t zDesc,
				const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem,
				avActivationType_t activation)
		{
			ConvCall call;
			const avStatus_t st = prepare_conv(context, config, alpha1, xDesc, xMem, wDesc, wMem, bDesc, bMem, alpha2, zDesc, zMem, beta, yDesc, yMem, call);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			/* 16-bit tensors: the one-kernel Winograd that transforms along rows only, where its shapes and the layer's size allow
			 * (a 256 x 15 x 15 x 128 -> 128 layer in bf16: 16 us against 43 us in the kernel that transforms in both directions) */
			if (rows_winograd_pays(call, activation))
			{
				const avStatus_t rs = run_rows_winograd(call, wMem, yMem, activation);
				if (rs != AVOCADO_STATUS_NOT_SUPPORTED)
					return rs; /* (BAD_ALLOC included: the entry reports a cold cache under capture as it always did) */
			}
			return run_fused_winograd(call, wMem, yMem, activation);
		}

		avStatus_t avhipConvolutionWinogradFusedForwardNoAlloc(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const void *alpha1,
				const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem,
				const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2, const avTensorDescriptor_t zDesc,
				const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem,
				avActivationType_t activation)
		{
			ConvCall call;
			const avStatus_t st = prepare_conv(context, config, alpha1, xDesc, xMem, wDesc, wMem, bDesc, bMem, alpha2, zDesc, zMem, beta, yDesc, yMem, call);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			const ConvProblem &p = call.problem;
			if (!fused_winograd_applicable(p))
				return AVOCADO_STATUS_NOT_SUPPORTED;
			if (call.bias != nullptr && call.bias_dtype != AVOCADO_DTYPE_FLOAT32)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			const avDataType_t mat_dtype = (p.w_dtype == AVOCADO_DTYPE_FLOAT32) ? AVOCADO_DTYPE_FLOAT32 : AVOCADO_DTYPE_FLOAT16;
			const av_int64 u_bytes = static_cast<av_int64>(16) * p.shape.K * p.shape.C * size_of(mat_dtype);
			if (u_bytes > static_cast<av_int64>(AVHIP_NOALLOC_SCRATCH_BYTES))
				return AVOCADO_STATUS_NOT_SUPPORTED; /* the transformed weights do not fit the fixed scratch array */
			void *U = nullptr; /* prepare_conv made the context's device current */
			const avStatus_t ss = noalloc_scratch_pointer(call.ctx.device, &U);
			if (ss != AVOCADO_STATUS_SUCCESS)
				return ss;
			/* the transform overwrites all of [16, K, C], so nothing of the previous call's contents is read */
			int rc = avhip_winograd_weight_transform(call.ctx.stream, p.w_dtype, mat_dtype, 2, 3, p.shape.mode, call.w->data, U, p.shape.K, p.shape.C);
			if (rc != 0)
				return from_launcher(rc);
			touch(yMem);
			rc = avhip_conv2d_winograd_fused(call.ctx.stream, p.x_dtype, &p.shape, call.x->data, U, call.bias, call.z, call.y->data, call.alpha1,
					call.alpha2, call.beta, activation);
			return from_launcher(rc);
		}

		avStatus_t avhipConvolutionRequantForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const avTensorDescriptor_t xDesc,
				const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem, const avTensorDescriptor_t bDesc,
				const avMemoryDescriptor_t bMem, const avTensorDescriptor_t scaleDesc, const avMemoryDescriptor_t scaleMem, const avTensorDescriptor_t yDesc,
				avMemoryDescriptor_t yMem, avActivationType_t activation)
		{
			ConvCall call;
			const avStatus_t st = prepare_conv(context, config, nullptr, xDesc, xMem, wDesc, wMem, bDesc, bMem, nullptr, 0, 0, nullptr, yDesc, yMem, call);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			const Tensor *sc = get_tensor(scaleDesc);
			Memory *sm = get_memory(scaleMem);
			if (sc == nullptr || sc->dtype != AVOCADO_DTYPE_FLOAT32 || sc->volume() != call.problem.shape.K || !fits(sm, sc->volume() * 4))
				return AVOCADO_STATUS_BAD_PARAM;
			if (call.problem.x_dtype != AVOCADO_DTYPE_INT8 || call.problem.y_dtype != AVOCADO_DTYPE_INT8)
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			return run_implicit_gemm(call, yMem, activation, reinterpret_cast<const float*>(sm->data));
		}

		avStatus_t cudaWinogradWeightTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
				const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem, const avTensorDescriptor_t matricesDesc, avMemoryDescriptor_t matricesMem)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Convolution *conv = get_convolution(config);
			const Tensor *w = get_tensor(wDesc), *mx = get_tensor(matricesDesc);
			if (conv == nullptr || w == nullptr || mx == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (!is_floating(w->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (w->nb_dims != 4 || mx->nb_dims != 3)
				return AVOCADO_STATUS_NOT_SUPPORTED;
			const int r = w->dim[1];
			if (!is_conv(r, *w) || !winograd_supported(r, transformSize))
				return AVOCADO_STATUS_NOT_SUPPORTED;
			if (!matrix_dtype_ok(w->dtype, mx->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			const int t = transformSize + r - 1;
			if (mx->dim[0] != t * t || mx->dim[1] != w->dim[0] || mx->dim[2] != w->dim[3])
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *wm = get_memory(wMem), *mm = get_memory(matricesMem);
			if (!fits(wm, w->volume() * size_of(w->dtype)) || !fits(mm, mx->volume() * size_of(mx->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(matricesMem);
			const int invert = (conv->mode == AVOCADO_CROSS_CORRELATION_MODE) ? 1 : 0;
			return from_launcher(avhip_winograd_weight_transform(ctx.stream, w->dtype, mx->dtype, transformSize, r, invert, wm->data, mm->data, w->dim[0],
					w->dim[3]));
		}

		avStatus_t cudaWinogradInputTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
				const avTensorDescriptor_t wDesc, const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t matricesDesc,
				avMemoryDescriptor_t matricesMem)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Convolution *conv = get_convolution(config);
			const Tensor *w = get_tensor(wDesc), *x = get_tensor(xDesc), *mx = get_tensor(matricesDesc);
			if (conv == nullptr || w == nullptr || x == nullptr || mx == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (!is_floating(x->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (w->nb_dims != 4 || x->nb_dims != 4 || mx->nb_dims != 3)
				return AVOCADO_STATUS_NOT_SUPPORTED;
			const int r = w->dim[1];
			if (!is_conv(r, *w) || !winograd_supported(r, transformSize))
				return AVOCADO_STATUS_NOT_SUPPORTED;
			if (!matrix_dtype_ok(x->dtype, mx->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			const int m = transformSize, t = m + r - 1;
			const av_int64 tiles = static_cast<av_int64>(x->dim[0]) * ((x->dim[1] + m - 1) / m) * ((x->dim[2] + m - 1) / m);
			if (mx->dim[0] != t * t || mx->dim[1] != tiles || mx->dim[2] != x->dim[3])
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *xm = get_memory(xMem), *mm = get_memory(matricesMem);
			if (!fits(xm, x->volume() * size_of(x->dtype)) || !fits(mm, mx->volume() * size_of(mx->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(matricesMem);
			return from_launcher(avhip_winograd_input_transform(ctx.stream, x->dtype, mx->dtype, m, r, xm->data, mm->data, x->dim[0], x->dim[1], x->dim[2],
					x->dim[3], conv->padding[0], conv->padding[1], padding_value_or_null(conv)));
		}

		avStatus_t cudaWinogradOutputTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
				const avTensorDescriptor_t wDesc, const void *alpha1, const avTensorDescriptor_t matricesDesc, const avMemoryDescriptor_t matricesMem,
				const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem, const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem,
				const void *alpha2, const avTensorDescriptor_t zDesc, const avMemoryDescriptor_t zMem, const void *beta, avActivationType_t activation)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Tensor *w = get_tensor(wDesc), *y = get_tensor(yDesc), *mx = get_tensor(matricesDesc);
			if (get_convolution(config) == nullptr || w == nullptr || y == nullptr || mx == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (!is_floating(y->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (w->nb_dims != 4 || y->nb_dims != 4 || mx->nb_dims != 3)
				return AVOCADO_STATUS_NOT_SUPPORTED;
			const int r = w->dim[1];
			if (!is_conv(r, *w) || !winograd_supported(r, transformSize))
				return AVOCADO_STATUS_NOT_SUPPORTED;
			if (!matrix_dtype_ok(y->dtype, mx->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			const int m = transformSize, t = m + r - 1;
			const av_int64 tiles = static_cast<av_int64>(y->dim[0]) * ((y->dim[1] + m - 1) / m) * ((y->dim[2] + m - 1) / m);
			if (mx->dim[0] != t * t || mx->dim[1] != tiles || mx->dim[2] != y->dim[3])
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *ym = get_memory(yMem), *mm = get_memory(matricesMem);
			const av_int64 ybytes = y->volume() * size_of(y->dtype);
			if (!fits(ym, ybytes) || !fits(mm, mx->volume() * size_of(mx->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
			char *bias = pointer_of(bMem), *z = pointer_of(zMem);
			const avDataType_t bias_type = (y->dtype == AVOCADO_DTYPE_FLOAT64) ? AVOCADO_DTYPE_FLOAT64 : AVOCADO_DTYPE_FLOAT32;
			if (bias != nullptr)
			{
				const Tensor *b = get_tensor(bDesc);
				if (b == nullptr || b->volume() != y->dim[3] || !fits(get_memory(bMem), b->volume() * size_of(bias_type)))
					return AVOCADO_STATUS_BAD_PARAM;
				if (b->dtype != bias_type)
					return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			}
			if (z != nullptr)
			{
				const Tensor *zd = get_tensor(zDesc);
				if (zd == nullptr || zd->volume() != y->volume() || zd->dtype != y->dtype || !fits(get_memory(zMem), ybytes))
					return AVOCADO_STATUS_BAD_PARAM;
			}
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(yMem);
			return from_launcher(avhip_winograd_output_transform(ctx.stream, y->dtype, mx->dtype, m, r, mm->data, ym->data, bias, z, y->dim[0], y->dim[1],
					y->dim[2], y->dim[3], scalar_or(alpha1, y->dtype, 1.0), scalar_or(alpha2, y->dtype, 1.0), scalar_or(beta, y->dtype, 0.0), activation));
		}

		avStatus_t cudaWinogradGradientTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize,
				const avTensorDescriptor_t wDesc, const avTensorDescriptor_t dyDesc, const avMemoryDescriptor_t dyMem, const avTensorDescriptor_t matricesDesc,
				avMemoryDescriptor_t matricesMem)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Tensor *w = get_tensor(wDesc), *dy = get_tensor(dyDesc), *mx = get_tensor(matricesDesc);
			if (get_convolution(config) == nullptr || w == nullptr || dy == nullptr || mx == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (!is_floating(dy->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (w->nb_dims != 4 || dy->nb_dims != 4 || mx->nb_dims != 3)
				return AVOCADO_STATUS_NOT_SUPPORTED;
			const int r = w->dim[1];
			if (!is_conv(r, *w) || !winograd_supported(r, transformSize))
				return AVOCADO_STATUS_NOT_SUPPORTED;
			if (!matrix_dtype_ok(dy->dtype, mx->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			const int m = transformSize, t = m + r - 1;
			const av_int64 tiles = static_cast<av_int64>(dy->dim[0]) * ((dy->dim[1] + m - 1) / m) * ((dy->dim[2] + m - 1) / m);
			if (mx->dim[0] != t * t || mx->dim[1] != tiles || mx->dim[2] != dy->dim[3])
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *dm = get_memory(dyMem), *mm = get_memory(matricesMem);
			if (!fits(dm, dy->volume() * size_of(dy->dtype)) || !fits(mm, mx->volume() * size_of(mx->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(matricesMem);
			return from_launcher(avhip_winograd_gradient_transform(ctx.stream, dy->dtype, mx->dtype, m, r, dm->data, mm->data, dy->dim[0], dy->dim[1],
					dy->dim[2], dy->dim[3]));
		}

		avStatus_t cudaWinogradUpdateTransform(avContextDescriptor_t context, const avConvolutionDescriptor_t config, int transformSize, const void *alpha,
				const avTensorDescriptor_t matricesDesc, const avMemoryDescriptor_t matricesMem, const void *beta, const avTensorDescriptor_t dwDesc,
				avMemoryDescriptor_t dwMem)
		{
			Context ctx;
			if (!get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			const Tensor *dw = get_tensor(dwDesc), *mx = get_tensor(matricesDesc);
			if (get_convolution(config) == nullptr || dw == nullptr || mx == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			if (!is_floating(dw->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			if (dw->nb_dims != 4 || mx->nb_dims != 3)
				return AVOCADO_STATUS_NOT_SUPPORTED;
			const int r = dw->dim[1];
			if (!is_conv(r, *dw) || !winograd_supported(r, transformSize))
				return AVOCADO_STATUS_NOT_SUPPORTED;
			if (!matrix_dtype_ok(dw->dtype, mx->dtype))
				return AVOCADO_STATUS_UNSUPPORTED_DATATYPE;
			const int t = transformSize + r - 1;
			if (mx->dim[0] != t * t || mx->dim[1] != dw->dim[0] || mx->dim[2] != dw->dim[3])
				return AVOCADO_STATUS_BAD_PARAM;
			Memory *wm = get_memory(dwMem), *mm = get_memory(matricesMem);
			if (!fits(wm, dw->volume() * size_of(dw->dtype)) || !fits(mm, mx->volume() * size_of(mx->dtype)))
				return AVOCADO_STATUS_BAD_PARAM;
			if (hipSetDevice(ctx.device) != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			touch(dwMem);
			return from_launcher(avhip_winograd_update_transform(ctx.stream, dw->dtype, mx->dtype, transformSize, r, mm->data, wm->data, dw->dim[0],
					dw->dim[3], scalar_or(alpha, dw->dtype, 1.0), scalar_or(beta, dw->dtype, 0.0)));
		}

		avStatus_t cudaGetConvolutionWorkspaceSize(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const avTensorDescriptor_t xDesc,
				const avTensorDescriptor_t wDesc, const avTensorDescriptor_t bDesc, av_int64 *result)
		{
			(void) bDesc;
			Context ctx;
			if (!get_context(context, ctx) || result == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			const Convolution *conv = get_convolution(config);
			const Tensor *x = get_tensor(xDesc), *w = get_tensor(wDesc);
			if (conv == nullptr || x == nullptr || w == nullptr || x->nb_dims != 4 || w->nb_dims != 4)
				return AVOCADO_STATUS_BAD_PARAM;
			/* output extent of a convolution whose offset padding is mirrored at the far edge */
			Tensor y = *x;
			y.dim[3] = w->dim[0];
			for (int i = 0; i < 2; i++)
			{
				const int extent = (w->dim[1 + i] - 1) * conv->dilation[i] + 1;
				if (conv->strides[i] <= 0 || conv->dilation[i] <= 0)
					return AVOCADO_STATUS_BAD_PARAM;
				y.dim[1 + i] = (x->dim[1 + i] - 2 * conv->padding[i] - extent) / conv->strides[i] + 1;
			}
			ConvProblem p;
			const avStatus_t st = make_problem(conv, x, w, &y, p);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			NonFusedPlan plan;
			result[0] = (nonfused_plan(p, plan) && (nonfused_preferred(p, plan) || !fused_winograd_applicable(p))) ? plan.total : 0;
			/* what the split-k plan of the implicit GEMM would take, for layers that go there */
			result[0] = std::max<av_int64>(result[0], split_k_bytes(p));
			return AVOCADO_STATUS_SUCCESS;
		}

		avStatus_t cudaConvolutionBiasActivationForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const void *alpha1,
				const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem,
				const avTensorDescriptor_t bDesc, const avMemoryDescriptor_t bMem, const void *alpha2, const avTensorDescriptor_t zDesc,
				const avMemoryDescriptor_t zMem, const void *beta, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem,
				const avActivationType_t activation, avMemoryDescriptor_t workspaceMem)
		{
			ConvCall call;
			const avStatus_t st = prepare_conv(context, config, alpha1, xDesc, xMem, wDesc, wMem, bDesc, bMem, alpha2, zDesc, zMem, beta, yDesc, yMem, call);
			if (st != AVOCADO_STATUS_SUCCESS)
				return st;
			const ConvProblem &p = call.problem;
			const bool bias_fp32 = call.bias == nullptr || call.bias_dtype == AVOCADO_DTYPE_FLOAT32;
			/* 3x3 / stride 1 on fp32 tensors with enough channels to fill the matrix cores: fused Winograd, whose 2.25-fold saving
			 * of multiplications is worth more than its transform work at the fp32 MFMA rate.  At the 16-bit MFMA rate the
			 * matrix cores are not what bounds the convolution and the direct image-tile kernel is measurably faster (24 us against
			 * 43 us on a 256 x 15 x 15 x 128 -> 128 layer in bf16). */
			/* its workgroups cover 16 x 16 pixels x 128 filters: a problem with too few of them is left to the implicit-GEMM
			 * kernels, which can cut it finer */
			const av_int64 fused_workgroups = static_cast<av_int64>(p.shape.N) * ((p.shape.Ho + 15) / 16) * ((p.shape.Wo + 15) / 16)
					* ((p.shape.K + 127) / 128);
			NonFusedPlan plan;
			Memory *ws = get_memory(workspaceMem);
			/* few output pixels and a long k: where the fused Winograd kernel does not pay (below), the implicit GEMM with k split
			 * across workgroups comes first (fp32 3x3 512->512 on 32 images of 7x7: 86 us against 340 us) */
			/* the fused kernel pays where its workgroups (one per compute unit) cover most of the chip and its 16 x 16 tiles are
			 * mostly image: at 128 workgroups it loses to the implicit GEMM (3x3 128->128 on 32 images of 28 x 28: 96 against 81 us),
			 * at 256 it wins (77 against 146 us on 64 images); on 7 x 7 images, a fifth of a tile, it takes twice the time of the
			 * implicit GEMM */
			const double fused_fill = static_cast<double>(p.shape.Ho) * p.shape.Wo / (((p.shape.Ho + 15) / 16 * 16.0) * ((p.shape.Wo + 15) / 16 * 16.0));
			const bool fused_pays = fused_workgroups >= 160 && fused_fill >= 0.5;
			/* 16-bit 3x3 layers on small images: row-wise Winograd (BAD_ALLOC: capturing with a cold cache; NOT_SUPPORTED:
			 * alignment; either way nothing was launched and the direct kernels take over) */
			if (rows_winograd_pays(call, activation))
			{
				const avStatus_t rs = run_rows_winograd(call, wMem, yMem, activation);
				if (rs != AVOCADO_STATUS_NOT_SUPPORTED && rs != AVOCADO_STATUS_BAD_ALLOC)
					return rs;
			}
			if (strided_kernel_pays(call, activation))
			{
				const avStatus_t rs = run_strided_kernel(call, wMem, yMem, activation);
				if (rs != AVOCADO_STATUS_NOT_SUPPORTED && rs != AVOCADO_STATUS_BAD_ALLOC)
					return rs;
			}
			if (pointwise_block_pays(call, activation))
			{
				const avStatus_t rs = run_pointwise_block(call, wMem, yMem, activation);
				if (rs != AVOCADO_STATUS_NOT_SUPPORTED && rs != AVOCADO_STATUS_BAD_ALLOC)
					return rs;
			}
			if (!fused_pays)
			{
				const avStatus_t ss = run_split_k(call, ws, workspaceMem, yMem, activation);
				if (ss != AVOCADO_STATUS_NOT_SUPPORTED)
					return ss;
			}
			const bool nonfused_ready = nonfused_plan(p, plan) && bias_fp32 && p.shape.C >= 32 && p.shape.K >= 32 && ws != nullptr && ws->data != nullptr
					&& ws->size >= plan.total && reinterpret_cast<uintptr_t>(ws->data) % 256 == 0;
			/* AVOCADO_STATUS_BAD_ALLOC from a Winograd plan means that the stream is capturing and the transformed weights are not
			 * in the library's cache yet (nothing was launched): the implicit-GEMM plan needs none and takes over. */
			if (nonfused_ready && nonfused_preferred(p, plan))
			{
				const avStatus_t ns = run_nonfused_winograd(call, plan, ws, wMem, workspaceMem, yMem, activation);
				if (ns != AVOCADO_STATUS_BAD_ALLOC)
					return ns;
			}
			else if (fused_winograd_applicable(p) && p.x_dtype == AVOCADO_DTYPE_FLOAT32 && bias_fp32 && p.shape.C >= 32 && p.shape.K >= 32
					&& p.shape.Ho == p.shape.H && p.shape.Wo == p.shape.W && fused_pays)
			{
				const avStatus_t fs = run_fused_winograd(call, wMem, yMem, activation);
				if (fs != AVOCADO_STATUS_NOT_SUPPORTED && fs != AVOCADO_STATUS_BAD_ALLOC)
					return fs;
				if (fs == AVOCADO_STATUS_NOT_SUPPORTED && nonfused_ready)
				{
					const avStatus_t ns = run_nonfused_winograd(call, plan, ws, wMem, workspaceMem, yMem, activation);
					if (ns != AVOCADO_STATUS_BAD_ALLOC)
						return ns;
				}
			}
			else if (nonfused_ready)
			{
				const avStatus_t ns = run_nonfused_winograd(call, plan, ws, wMem, workspaceMem, yMem, activation);
				if (ns != AVOCADO_STATUS_BAD_ALLOC)
					return ns;
			}
			const avStatus_t ss = run_split_k(call, ws, workspaceMem, yMem, activation);
			if (ss != AVOCADO_STATUS_NOT_SUPPORTED)
				return ss;
			return run_implicit_gemm(call, yMem, activation, nullptr);
		}

		avStatus_t cudaConvolutionForward(avContextDescriptor_t context, const avConvolutionDescriptor_t config, const void *alpha,
				const avTensorDescriptor_t xDesc, const avMemoryDescriptor_t xMem, const avTensorDescriptor_t wDesc, const avMemoryDescriptor_t wMem,
				const void *beta, const avTensorDescriptor_t yDesc, avMemoryDescriptor_t yMem, avMemoryDescriptor_t workspaceMem)
		{
			return cudaConvolutionBiasActivationForward(context, config, alpha, xDesc, xMem, wDesc, wMem, 0, 0, nullptr, 0, 0, beta, yDesc, yMem,
					AVOCADO_ACTIVATION_LINEAR, workspaceMem);
		}

		/* -------------------------------------------------------------------------------------------------- additions */
		avStatus_t avhipGetContextStream(avContextDescriptor_t context, void **stream)
		{
			Context ctx;
			if (stream == nullptr || !get_context(context, ctx))
				return AVOCADO_STATUS_BAD_PARAM;
			stream[0] = ctx.stream;
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t avhipGetMemoryPointer(avMemoryDescriptor_t mem, void **pointer)
		{
			Memory *m = get_memory(mem);
			if (pointer == nullptr || m == nullptr)
				return AVOCADO_STATUS_BAD_PARAM;
			pointer[0] = m->data;
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t avhipInvalidateCaches(void)
		{
			if (hipDeviceSynchronize() != hipSuccess)
				return AVOCADO_STATUS_EXECUTION_FAILED;
			weight_cache().clear();
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t avhipSetWeightCacheBudget(av_int64 bytes, av_int64 *previous)
		{
			if (bytes < 0)
				return AVOCADO_STATUS_BAD_PARAM;
			WeightCache &cache = weight_cache();
			std::lock_guard<std::mutex> lock(cache.mutex);
			if (previous != nullptr)
				previous[0] = static_cast<av_int64>(cache.budget);
			cache.budget = static_cast<size_t>(bytes);
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t avhipWeightCachePolicyProbe(int count, const av_int64 *bytes, const av_int64 *last_use, const int *flags, av_int64 budget, av_int64 incoming,
				int *evicted)
		{
			if (count < 0 || bytes == nullptr || last_use == nullptr || flags == nullptr || evicted == nullptr || budget < 0 || incoming < 0)
				return AVOCADO_STATUS_BAD_PARAM;
			WeightCache model; /* the same object the library keeps, filled with entries that own nothing */
			model.budget = static_cast<size_t>(budget);
			for (int i = 0; i < count; i++)
			{
				WeightEntry e;
				e.bytes = static_cast<size_t>(bytes[i]);
				e.last_use = static_cast<uint64_t>(last_use[i]);
				e.pinned = (flags[i] & 1) != 0;
				e.in_use = (flags[i] & 2) != 0 ? 1 : 0;
				model.entries.emplace(WeightKey { static_cast<uint64_t>(i), 0, 0, 0, 0, 0, 0 }, e);
				model.total += e.bytes;
			}
			std::vector<WeightEntry> victims;
			model.make_room(static_cast<size_t>(incoming), victims);
			for (int i = 0; i < count; i++)
				evicted[i] = model.entries.count(WeightKey { static_cast<uint64_t>(i), 0, 0, 0, 0, 0, 0 }) == 0 ? 1 : 0;
			return AVOCADO_STATUS_SUCCESS;
		}
		avStatus_t avhipGetWeightCacheState(av_int64 *entries, av_int64 *bytes, av_int64 *transforms)
		{
			WeightCache &cache = weight_cache();
			std::lock_guard<std::mutex> lock(cache.mutex);
			if (entries != nullptr)
				entries[0] = static_cast<av_int64>(cache.entries.size());
			if (bytes != nullptr)
				bytes[0] = static_cast<av_int64>(cache.total);
			if (transforms != nullptr)
				transforms[0] = static_cast<av_int64>(cache.transforms);
			return AVOCADO_STATUS_SUCCESS;
		}
	} /* namespace backend */
} /* namespace avocado */
