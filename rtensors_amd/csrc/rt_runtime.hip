// Context, stream, caching device allocator, host<->device transfers, events.
// Stands where backend/cuda.rs:38-185 and 668-836 (cudarc context, CudaSlice alloc/copy, sync-on-read) stand in
// the reference; written directly against the HIP runtime.
#include "rt_common.h"

#include <atomic>
#include <condition_variable>
#include <string>
#include <thread>

// ---- error plumbing ---------------------------------------------------------------------------------------------
static thread_local char g_err[512] = "";

int32_t rt_fail(int32_t status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int32_t rt_hip_fail(hipError_t e, const char* what) {
    if (e == hipErrorOutOfMemory) return rt_fail(RT_E_OOM, "%s: %s", what, hipGetErrorString(e));
    return rt_fail(RT_E_HIP, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
}

extern "C" const char* rt_last_error(void) { return g_err; }

extern "C" const char* rt_status_name(int32_t s) {
    switch (s) {
        case RT_OK: return "RT_OK";
        case RT_E_INVALID: return "RT_E_INVALID";
        case RT_E_DTYPE: return "RT_E_DTYPE";
        case RT_E_OUT_OF_BOUNDS: return "RT_E_OUT_OF_BOUNDS";
        case RT_E_HIP: return "RT_E_HIP";
        case RT_E_OOM: return "RT_E_OOM";
        case RT_E_RANK: return "RT_E_RANK";
        case RT_E_ARITH: return "RT_E_ARITH";
        case RT_E_WRONG_DIMS: return "RT_E_WRONG_DIMS";
        case RT_E_SIZE_MISMATCH: return "RT_E_SIZE_MISMATCH";
    }
    return "RT_E_UNKNOWN";
}

extern "C" int32_t rt_dtype_size(int32_t dtype) { return rt_elem_size(dtype); }

extern "C" int32_t rt_device_count(int32_t* out) {
    if (!out) return rt_fail(RT_E_INVALID, "rt_device_count: null out");
    int n = 0;
    RT_HIP(hipGetDeviceCount(&n));
    *out = n;
    return RT_OK;
}

// ---- context ------------------------------------------------------------------------------------------------------
int32_t rt_ctx_enter(rt_ctx* ctx) {
    if (!ctx) return rt_fail(RT_E_INVALID, "null context");
    RT_HIP(hipSetDevice(ctx->device));
    return RT_OK;
}

extern "C" int32_t rt_ctx_create(int32_t device, rt_ctx** out) {
    if (!out) return rt_fail(RT_E_INVALID, "rt_ctx_create: null out");
    *out = nullptr;
    int n = 0;
    RT_HIP(hipGetDeviceCount(&n));
    if (device == -1) {
        device = 0;
        if (const char* e = getenv("RT_HIP_DEVICE")) {
            char* end = nullptr;
            const long v = strtol(e, &end, 10);
            if (end == e || *end != '\0' || v < 0 || v > 1 << 20) return rt_fail(RT_E_INVALID, "rt_ctx_create: RT_HIP_DEVICE='%s' is not a device index", e);
            device = (int32_t)v;
        }
    }
    if (device < 0 || device >= n) return rt_fail(RT_E_INVALID, "rt_ctx_create: device %d of %d", device, n);
    RT_HIP(hipSetDevice(device));
    rt_ctx* c = new rt_ctx();
    c->device = device;
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);   // default priority
    if (e != hipSuccess) { delete c; return rt_hip_fail(e, "hipStreamCreateWithFlags"); }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0) c->num_cus = prop.multiProcessorCount;
    e = hipMalloc((void**)&c->flag_dev, 256);
    if (e != hipSuccess) { (void)hipStreamDestroy(c->stream); delete c; return rt_hip_fail(e, "hipMalloc(flag)"); }
    e = hipMemset(c->flag_dev, 0, 256);
    if (e != hipSuccess) { (void)hipFree(c->flag_dev); (void)hipStreamDestroy(c->stream); delete c; return rt_hip_fail(e, "hipMemset(flag)"); }
    c->fault_dev = c->flag_dev + 16;                         // its own 64-byte piece of the block
    // the device address of the library's built-in workspace, looked up here so that the entry point that allocates nothing makes no
    // runtime query of its own (a symbol lookup is not safe under stream capture)
    const int32_t ws = rt_static_scratch_init(device, &c->static_scratch);
    if (ws != RT_OK) { (void)hipFree(c->flag_dev); (void)hipStreamDestroy(c->stream); delete c; return ws; }
    *out = c;
    return RT_OK;
}

extern "C" int32_t rt_ctx_destroy(rt_ctx* ctx) {
    RT_TRY(rt_ctx_enter(ctx));
    {
        CtxGuard g(ctx);
        (void)hipStreamSynchronize(ctx->stream);
        for (auto& kv : ctx->free_blocks) (void)hipFree(kv.second);
        for (auto& kv : ctx->live) (void)hipFree(kv.first);
        if (ctx->scratch) (void)hipFree(ctx->scratch);
        if (ctx->blas && ctx->blas_destroy) (void)ctx->blas_destroy(ctx->blas);
        for (int i = 0; i < 4; ++i) {
            if (ctx->stage[i]) (void)hipHostFree(ctx->stage[i]);
            if (ctx->stage_ev[i]) (void)hipEventDestroy(ctx->stage_ev[i]);
        }
        if (ctx->flag_dev) (void)hipFree(ctx->flag_dev);
        (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
    return RT_OK;
}

__global__ void rt_clear_word_kernel(int32_t* p) { *p = 0; }

int32_t rt_take_fault(rt_ctx* ctx) {
    if (!ctx->fault_pending) return RT_OK;
    ctx->fault_pending = false;
    int32_t host = 0;
    RT_HIP(hipMemcpyAsync(&host, ctx->fault_dev, sizeof(host), hipMemcpyDeviceToHost, ctx->stream));
    RT_HIP(hipStreamSynchronize(ctx->stream));
    if (!host) return RT_OK;
    hipLaunchKernelGGL(rt_clear_word_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->fault_dev);
    RT_HIP(hipGetLastError());
    return rt_fail(RT_E_ARITH, "an integer division enqueued earlier met a zero divisor or MIN / -1 (the reference panics there); "
                               "the elements concerned hold 0 / MIN");
}

extern "C" int32_t rt_sync(rt_ctx* ctx) {
    RT_TRY(rt_ctx_enter(ctx));
    RT_HIP(hipStreamSynchronize(ctx->stream));
    CtxGuard g(ctx);
    return rt_take_fault(ctx);
}

// ---- caching allocator ---------------------------------------------------------------------------------------------
// Size classes: multiples of 512 B below 1 MiB, multiples of 2 MiB above.  A freed block keeps its capacity and is
// reused for the next request of the same class; nothing is split, so there is no fragmentation to manage, and a
// training step that allocates the same shapes every iteration reaches a state with no hipMalloc at all.
static size_t size_class(size_t bytes) {
    if (bytes == 0) bytes = 1;
    if (bytes < (1u << 20)) return (bytes + 511) & ~(size_t)511;
    const size_t g = (size_t)2 << 20;
    return (bytes + g - 1) / g * g;
}

int32_t rt_alloc_bytes(rt_ctx* ctx, size_t bytes, void** out) {
    size_t cap = size_class(bytes);
    auto it = ctx->free_blocks.find(cap);
    if (it != ctx->free_blocks.end()) {
        *out = it->second;
        ctx->free_blocks.erase(it);
        ctx->bytes_cached -= cap;
    } else {
        void* p = nullptr;
        hipError_t e = hipMalloc(&p, cap);
        if (e == hipErrorOutOfMemory && !ctx->free_blocks.empty()) {
            // give cached blocks back to the driver and retry once
            (void)hipGetLastError();
            (void)hipStreamSynchronize(ctx->stream);
            for (auto& kv : ctx->free_blocks) (void)hipFree(kv.second);
            ctx->free_blocks.clear();
            ctx->bytes_cached = 0;
            e = hipMalloc(&p, cap);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            *out = nullptr;
            return rt_hip_fail(e, "hipMalloc");
        }
        ctx->device_allocs += 1;
        *out = p;
    }
    ctx->live[*out] = cap;
    ctx->bytes_in_use += cap;
    return RT_OK;
}

int32_t rt_free_locked(rt_ctx* ctx, void* p) {
    auto it = ctx->live.find(p);
    if (it == ctx->live.end()) return rt_fail(RT_E_INVALID, "rt_free: %p was not allocated by this context", p);
    size_t cap = it->second;
    ctx->live.erase(it);
    ctx->bytes_in_use -= cap;
    ctx->free_blocks.emplace(cap, p);
    ctx->bytes_cached += cap;
    return RT_OK;
}

int32_t rt_scratch(rt_ctx* ctx, size_t bytes, void** out) {
    if (ctx->fixed_only) {
        if (bytes > ctx->fixed_scratch_bytes)
            return rt_fail(RT_E_INVALID, "this reduction needs %zu bytes of partial results; the built-in workspace of the entry point "
                           "that allocates nothing holds %zu (use rt_reduce_nd)", bytes, ctx->fixed_scratch_bytes);
        *out = ctx->fixed_scratch;
        return RT_OK;
    }
    if (bytes > ctx->scratch_bytes) {
        if (ctx->scratch) {
            RT_HIP(hipStreamSynchronize(ctx->stream));
            RT_HIP(hipFree(ctx->scratch));
            ctx->scratch = nullptr;
            ctx->scratch_bytes = 0;
        }
        size_t cap = size_class(bytes < (1u << 20) ? (1u << 20) : bytes);
        RT_HIP(hipMalloc(&ctx->scratch, cap));
        ctx->scratch_bytes = cap;
        ctx->device_allocs += 1;
    }
    *out = ctx->scratch;
    return RT_OK;
}

__global__ void rt_zero_kernel(uint4* p, size_t nvec) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < nvec; i += step) p[i] = make_uint4(0, 0, 0, 0);
}
// The zero fill of Backend::alloc for large blocks: one vector per lane in the write-only tiled order (512-lane blocks own 1 KiB
// pieces of 16 pages 64 KiB apart, see TileMap), non-temporal stores.  1 GiB: 0.279 ms with the grid-stride kernel above, 0.15 ms so.
__global__ __launch_bounds__(512) void rt_zero_tiled_kernel(rt_u32x4* p, size_t nvec, TileMap m) {
    size_t i;
    if (!rt_tile_index(m, blockIdx.x, 512, threadIdx.x, nvec, &i)) return;
    const rt_u32x4 z = {0u, 0u, 0u, 0u};
    __builtin_nontemporal_store(z, p + i);
}

// ---- host <-> device transfers ----------------------------------------------------------------------------------------
// A copy between device memory and ordinary (pageable) host memory goes through a ring of pinned staging buffers: the DMA
// engine moves chunk i between the device and slot i % 4 while four host threads copy another chunk between its slot and the
// caller's memory.  Measured on an MI355X host for 1 GiB: 50 GB/s down and 52 GB/s up, against 16 and 29 GB/s for
// hipMemcpy on the pageable pointer itself.  Transfers below kStagedMin go directly.
namespace {

constexpr size_t kStageBytes = (size_t)8 << 20;
constexpr int kStages = 4;
constexpr int kCopyThreads = 4;
constexpr size_t kStagedMin = (size_t)4 << 20;

// memcpy split over kCopyThreads threads: the caller takes the first part, kCopyThreads - 1 helpers the others.  The helpers
// are started by the first copy and live as long as the process (the pool is never destroyed).  A chunk takes ~0.1 ms, the
// same order as a condition-variable wake-up, so a helper first polls the generation counter for about that long after
// finishing a part and only then blocks; between transfers the helpers sleep.
class CopyPool {
  public:
    static CopyPool& get() {
        static CopyPool* pool = new CopyPool();
        return *pool;
    }
    void copy(char* dst, const char* src, size_t bytes) {
        std::lock_guard<std::mutex> user(user_mu_);
        if (!started_) {
            for (int i = 1; i < kCopyThreads; ++i) std::thread([this, i] { worker(i); }).detach();
            started_ = true;
        }
        size_t per = (bytes + kCopyThreads - 1) / kCopyThreads;
        per = (per + 63) & ~(size_t)63;
        dst_ = dst; src_ = src; bytes_ = bytes; per_ = per;
        pending_.store(kCopyThreads - 1, std::memory_order_relaxed);
        gen_.fetch_add(1, std::memory_order_release);          // publishes the task fields above
        { std::lock_guard<std::mutex> lk(mu_); }                // a helper is either before its predicate check or already waiting
        work_.notify_all();
        memcpy(dst, src, per < bytes ? per : bytes);
        for (unsigned spins = 0; pending_.load(std::memory_order_acquire) != 0; ++spins) {
            if (spins < kSpin) __builtin_ia32_pause(); else std::this_thread::yield();
        }
    }

  private:
    static constexpr unsigned kSpin = 20000;                    // ~0.1 ms of polling
    void worker(int idx) {
        uint64_t seen = 0;
        for (;;) {
            uint64_t g;
            for (unsigned spins = 0; (g = gen_.load(std::memory_order_acquire)) == seen; ++spins) {
                if (spins < kSpin) { __builtin_ia32_pause(); continue; }
                std::unique_lock<std::mutex> lk(mu_);
                work_.wait(lk, [&] { return gen_.load(std::memory_order_acquire) != seen; });
            }
            seen = g;
            const size_t o = (size_t)idx * per_;
            if (o < bytes_) memcpy(dst_ + o, src_ + o, per_ < bytes_ - o ? per_ : bytes_ - o);
            pending_.fetch_sub(1, std::memory_order_acq_rel);
        }
    }
    std::mutex user_mu_, mu_;
    std::condition_variable work_;
    std::atomic<uint64_t> gen_{0};
    std::atomic<int> pending_{0};
    char* dst_ = nullptr;
    const char* src_ = nullptr;
    size_t bytes_ = 0, per_ = 0;
    bool started_ = false;
};

int32_t ensure_staging(rt_ctx* ctx) {                      // caller holds ctx->mu
    for (int i = 0; i < kStages; ++i) {
        if (!ctx->stage[i]) RT_HIP(hipHostMalloc(&ctx->stage[i], kStageBytes, hipHostMallocDefault));
        if (!ctx->stage_ev[i]) RT_HIP(hipEventCreateWithFlags(&ctx->stage_ev[i], hipEventDisableTiming));
    }
    return RT_OK;
}

// device -> host, ordered after everything already on the stream; returns when the host buffer is complete
int32_t download(rt_ctx* ctx, void* host_dst, const void* dev_src, size_t bytes) {
    if (bytes < kStagedMin || ensure_staging(ctx) != RT_OK) {
        RT_HIP(hipMemcpyAsync(host_dst, dev_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
        RT_HIP(hipStreamSynchronize(ctx->stream));
        return RT_OK;
    }
    const size_t nch = (bytes + kStageBytes - 1) / kStageBytes;
    auto chunk_bytes = [&](size_t j) { return j + 1 < nch ? kStageBytes : bytes - j * kStageBytes; };
    auto issue = [&](size_t j) -> hipError_t {
        hipError_t e = hipMemcpyAsync(ctx->stage[j % kStages], (const char*)dev_src + j * kStageBytes, chunk_bytes(j), hipMemcpyDeviceToHost, ctx->stream);
        if (e == hipSuccess) e = hipEventRecord(ctx->stage_ev[j % kStages], ctx->stream);
        return e;
    };
    hipError_t e = hipSuccess;
    for (size_t j = 0; j < (size_t)kStages && j < nch && e == hipSuccess; ++j) e = issue(j);
    for (size_t j = 0; j < nch && e == hipSuccess; ++j) {
        e = hipEventSynchronize(ctx->stage_ev[j % kStages]);
        if (e != hipSuccess) break;
        CopyPool::get().copy((char*)host_dst + j * kStageBytes, (const char*)ctx->stage[j % kStages], chunk_bytes(j));
        if (j + kStages < nch) e = issue(j + kStages);
    }
    if (e != hipSuccess) {
        (void)hipStreamSynchronize(ctx->stream);
        return rt_hip_fail(e, "download");
    }
    return RT_OK;
}

// host -> device; returns when the host buffer may be reused and the data is in device memory
int32_t upload(rt_ctx* ctx, void* dev_dst, const void* host_src, size_t bytes) {
    if (bytes < kStagedMin || ensure_staging(ctx) != RT_OK) {
        RT_HIP(hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice, ctx->stream));
        RT_HIP(hipStreamSynchronize(ctx->stream));
        return RT_OK;
    }
    const size_t nch = (bytes + kStageBytes - 1) / kStageBytes;
    hipError_t e = hipSuccess;
    for (size_t j = 0; j < nch && e == hipSuccess; ++j) {
        const size_t n = j + 1 < nch ? kStageBytes : bytes - j * kStageBytes;
        const int slot = (int)(j % kStages);
        if (j >= (size_t)kStages) e = hipEventSynchronize(ctx->stage_ev[slot]);      // the slot's previous chunk has left it
        if (e != hipSuccess) break;
        CopyPool::get().copy((char*)ctx->stage[slot], (const char*)host_src + j * kStageBytes, n);
        e = hipMemcpyAsync((char*)dev_dst + j * kStageBytes, ctx->stage[slot], n, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipEventRecord(ctx->stage_ev[slot], ctx->stream);
    }
    hipError_t e2 = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) e = e2;
    if (e != hipSuccess) return rt_hip_fail(e, "upload");
    return RT_OK;
}

}  // namespace

// ---- device -> device copy ------------------------------------------------------------------------------------------------
// One 16-byte vector per lane, 128-lane blocks, non-temporal load and store: 6.5 TB/s for 1 GiB on MI355X, against 5.0 TB/s
// for hipMemcpyAsync(DeviceToDevice).  s and d point at the vector body, which starts on a 128-byte line of d; the source may be
// in any phase (16-byte loads at byte alignment).  The `head` bytes before the body and the `tail` bytes after it go to lanes of
// the first and the last block.
__global__ __launch_bounds__(256) void rt_copy_vec_kernel(const uint8_t* __restrict__ s, uint8_t* __restrict__ d, size_t nvec, uint32_t head, uint32_t tail,
                                                          TileMap m) {
    if (blockIdx.x == 0 && threadIdx.x < head) { const int64_t e = (int64_t)threadIdx.x - (int64_t)head; d[e] = s[e]; }
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x < tail) { const size_t e = nvec * 16 + threadIdx.x; d[e] = s[e]; }
    size_t i;
    if (!rt_tile_index(m, blockIdx.x, 256, threadIdx.x, nvec, &i)) return;          // a block owns a quarter of four pages (see TileMap)
    __builtin_nontemporal_store(rt_ld16u<uint8_t, true>(s + i * 16), reinterpret_cast<rt_u32x4*>(d) + i);
}

static int32_t device_copy(rt_ctx* ctx, void* dst, const void* src, size_t bytes) {      // caller holds ctx->mu
    if (!bytes) return RT_OK;
    const uintptr_t da = reinterpret_cast<uintptr_t>(dst);
    size_t head = (128 - (da & 127)) & 127;
    if (head > bytes) head = bytes;
    const size_t nvec = (bytes - head) / 16, tail = bytes - head - nvec * 16;
    const TileMap m = rt_make_tilemap((const uint8_t*)dst + head, nvec, 256);
    size_t blocks = rt_tilemap_blocks(m, nvec, 256);
    if (blocks < 1) blocks = 1;
    if (blocks > 0x7fffffffull) {
        RT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
        return RT_OK;
    }
    RT_TRY(rt_check_edges("copy", head, nvec, 16, tail, bytes, 256));
    hipLaunchKernelGGL(rt_copy_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const uint8_t*)src + head, (uint8_t*)dst + head, nvec,
                       (uint32_t)head, (uint32_t)tail, m);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

static int32_t checked_bytes(int32_t dtype, uint64_t len, size_t* bytes) {
    int es = rt_elem_size(dtype);
    if (es == 0) return rt_fail(RT_E_DTYPE, "unknown dtype code %d", dtype);
    if (len > (UINT64_MAX >> 5)) return rt_fail(RT_E_INVALID, "length %llu is too large", (unsigned long long)len);
    *bytes = (size_t)len * (size_t)es;
    return RT_OK;
}

static int32_t alloc_impl(rt_ctx* ctx, int32_t dtype, uint64_t len, void** out, bool zero) {
    if (!out) return rt_fail(RT_E_INVALID, "rt_alloc: null out");
    *out = nullptr;
    RT_TRY(rt_ctx_enter(ctx));
    size_t bytes = 0;
    RT_TRY(checked_bytes(dtype, len, &bytes));
    CtxGuard g(ctx);
    RT_TRY(rt_alloc_bytes(ctx, bytes, out));
    if (zero && bytes) {
        // whole size class is zeroed (capacity is a multiple of 512 B), by a fill kernel rather than a memset node
        size_t nvec = size_class(bytes) / 16;
        const TileMap m = rt_make_tilemap(*out, nvec, 512, 1024, 16, 65536);
        const size_t tiled_blocks = rt_tilemap_blocks(m, nvec, 512);
        if (nvec >= (1u << 16) && tiled_blocks <= 0x7fffffffull) {
            hipLaunchKernelGGL(rt_zero_tiled_kernel, dim3((unsigned)tiled_blocks), dim3(512), 0, ctx->stream, (rt_u32x4*)*out, nvec, m);
        } else {
            size_t blocks = (nvec + 255) / 256;
            if (blocks > (size_t)ctx->num_cus * 16) blocks = (size_t)ctx->num_cus * 16;
            hipLaunchKernelGGL(rt_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (uint4*)*out, nvec);
        }
        RT_HIP(hipGetLastError());
    }
    return RT_OK;
}

extern "C" int32_t rt_alloc(rt_ctx* ctx, int32_t dtype, uint64_t len, void** out) { return alloc_impl(ctx, dtype, len, out, true); }
extern "C" int32_t rt_alloc_uninit(rt_ctx* ctx, int32_t dtype, uint64_t len, void** out) { return alloc_impl(ctx, dtype, len, out, false); }

extern "C" int32_t rt_free(rt_ctx* ctx, void* buf) {
    if (!buf) return RT_OK;
    RT_TRY(rt_ctx_enter(ctx));
    CtxGuard g(ctx);
    return rt_free_locked(ctx, buf);
}

extern "C" int32_t rt_alloc_from_slice(rt_ctx* ctx, int32_t dtype, const void* host_src, uint64_t len, void** out) {
    if (!out) return rt_fail(RT_E_INVALID, "rt_alloc_from_slice: null out");
    *out = nullptr;
    if (!host_src && len) return rt_fail(RT_E_INVALID, "rt_alloc_from_slice: null source");
    RT_TRY(rt_ctx_enter(ctx));
    size_t bytes = 0;
    RT_TRY(checked_bytes(dtype, len, &bytes));
    CtxGuard g(ctx);
    RT_TRY(rt_alloc_bytes(ctx, bytes, out));
    if (bytes) {
        int32_t rc = upload(ctx, *out, host_src, bytes);              // the host slice may be dropped on return
        if (rc != RT_OK) { (void)rt_free_locked(ctx, *out); *out = nullptr; return rc; }
    }
    return RT_OK;
}

extern "C" int32_t rt_copy_from_slice(rt_ctx* ctx, int32_t dtype, void* dst, uint64_t dst_len, const void* host_src, uint64_t src_len) {
    RT_TRY(rt_ctx_enter(ctx));
    if (dst_len != src_len)
        return rt_fail(RT_E_SIZE_MISMATCH, "copy_from_slice: dst size %llu, src size %llu", (unsigned long long)dst_len, (unsigned long long)src_len);
    size_t bytes = 0;
    RT_TRY(checked_bytes(dtype, src_len, &bytes));
    if (!bytes) return RT_OK;
    if (!dst || !host_src) return rt_fail(RT_E_INVALID, "copy_from_slice: null pointer");
    CtxGuard g(ctx);
    return upload(ctx, dst, host_src, bytes);
}

extern "C" int32_t rt_copy_range_within(rt_ctx* ctx, int32_t dtype, void* dst, uint64_t dst_len, const void* src, uint64_t src_len,
                                        uint64_t dst_offset, uint64_t src_offset, uint64_t len) {
    RT_TRY(rt_ctx_enter(ctx));
    int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "unknown dtype code %d", dtype);
    if (dst_offset > dst_len || len > dst_len - dst_offset || src_offset > src_len || len > src_len - src_offset)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "copy_range_within: dst size %llu, src size %llu, dst_offset %llu, src_offset %llu, len %llu",
                       (unsigned long long)dst_len, (unsigned long long)src_len, (unsigned long long)dst_offset,
                       (unsigned long long)src_offset, (unsigned long long)len);
    if (!len) return RT_OK;
    if (!dst || !src) return rt_fail(RT_E_INVALID, "copy_range_within: null pointer");
    {
        const ByteSpan a = rt_run_span(dst, es, dst_offset, len), b = rt_run_span(src, es, src_offset, len);
        if (a.lo == b.lo) return RT_OK;                       // a range onto itself
        if (rt_spans_meet(a, b)) return rt_fail(RT_E_INVALID, "copy_range_within: the two ranges overlap");
    }
    CtxGuard g(ctx);
    return device_copy(ctx, (char*)dst + dst_offset * es, (const char*)src + src_offset * es, (size_t)len * es);
}

extern "C" int32_t rt_read(rt_ctx* ctx, int32_t dtype, const void* buf, uint64_t buf_len, uint64_t offset, void* out_value) {
    RT_TRY(rt_ctx_enter(ctx));
    int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "unknown dtype code %d", dtype);
    if (offset >= buf_len)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "Index %llu out of bounds for buffer of length %llu", (unsigned long long)offset, (unsigned long long)buf_len);
    if (!buf || !out_value) return rt_fail(RT_E_INVALID, "rt_read: null pointer");
    CtxGuard g(ctx);
    RT_HIP(hipMemcpyAsync(out_value, (const char*)buf + offset * es, es, hipMemcpyDeviceToHost, ctx->stream));
    RT_HIP(hipStreamSynchronize(ctx->stream));
    return rt_take_fault(ctx);
}

struct Cell16 { uint32_t w[4]; };

__global__ void rt_write_one_kernel(unsigned char* dst, Cell16 v, int bytes) {
    const unsigned char* s = (const unsigned char*)&v;
    for (int i = 0; i < bytes; ++i) dst[i] = s[i];
}

extern "C" int32_t rt_write(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, uint64_t offset, const void* value) {
    RT_TRY(rt_ctx_enter(ctx));
    int es = rt_elem_size(dtype);
    if (!es) return rt_fail(RT_E_DTYPE, "unknown dtype code %d", dtype);
    if (offset >= buf_len)
        return rt_fail(RT_E_OUT_OF_BOUNDS, "Index %llu out of bounds for buffer of length %llu", (unsigned long long)offset, (unsigned long long)buf_len);
    if (!buf || !value) return rt_fail(RT_E_INVALID, "rt_write: null pointer");
    Cell16 v = {{0, 0, 0, 0}};
    memcpy(&v, value, es);
    CtxGuard g(ctx);
    // the value travels as a kernel argument, so no host memory has to outlive this call
    hipLaunchKernelGGL(rt_write_one_kernel, dim3(1), dim3(1), 0, ctx->stream, (unsigned char*)buf + offset * es, v, es);
    RT_HIP(hipGetLastError());
    return RT_OK;
}

extern "C" int32_t rt_copy(rt_ctx* ctx, int32_t dtype, const void* src, uint64_t len, void** out) {
    if (!out) return rt_fail(RT_E_INVALID, "rt_copy: null out");
    *out = nullptr;
    RT_TRY(rt_ctx_enter(ctx));
    size_t bytes = 0;
    RT_TRY(checked_bytes(dtype, len, &bytes));
    if (!src && bytes) return rt_fail(RT_E_INVALID, "rt_copy: null source");
    CtxGuard g(ctx);
    RT_TRY(rt_alloc_bytes(ctx, bytes, out));
    if (bytes) {
        int32_t rc = device_copy(ctx, *out, src, bytes);
        if (rc != RT_OK) { (void)rt_free_locked(ctx, *out); *out = nullptr; return rc; }
    }
    return RT_OK;
}

extern "C" int32_t rt_dump(rt_ctx* ctx, int32_t dtype, const void* src, uint64_t len, void* host_dst) {
    RT_TRY(rt_ctx_enter(ctx));
    size_t bytes = 0;
    RT_TRY(checked_bytes(dtype, len, &bytes));
    if (!bytes) return RT_OK;
    if (!src || !host_dst) return rt_fail(RT_E_INVALID, "rt_dump: null pointer");
    CtxGuard g(ctx);
    RT_TRY(download(ctx, host_dst, src, bytes));
    return rt_take_fault(ctx);
}

// ---- events / stats -----------------------------------------------------------------------------------------------
struct rt_event { hipEvent_t ev; };

extern "C" int32_t rt_event_create(rt_ctx* ctx, rt_event** out) {
    if (!out) return rt_fail(RT_E_INVALID, "rt_event_create: null out");
    RT_TRY(rt_ctx_enter(ctx));
    rt_event* e = new rt_event();
    hipError_t r = hipEventCreate(&e->ev);
    if (r != hipSuccess) { delete e; return rt_hip_fail(r, "hipEventCreate"); }
    *out = e;
    return RT_OK;
}

extern "C" int32_t rt_event_record(rt_ctx* ctx, rt_event* ev) {
    RT_TRY(rt_ctx_enter(ctx));
    if (!ev) return rt_fail(RT_E_INVALID, "rt_event_record: null event");
    RT_HIP(hipEventRecord(ev->ev, ctx->stream));
    return RT_OK;
}

extern "C" int32_t rt_event_elapsed_ms(rt_ctx* ctx, rt_event* start, rt_event* stop, float* out_ms) {
    RT_TRY(rt_ctx_enter(ctx));
    if (!start || !stop || !out_ms) return rt_fail(RT_E_INVALID, "rt_event_elapsed_ms: null argument");
    RT_HIP(hipEventSynchronize(stop->ev));
    RT_HIP(hipEventElapsedTime(out_ms, start->ev, stop->ev));
    return RT_OK;
}

extern "C" int32_t rt_event_destroy(rt_ctx* ctx, rt_event* ev) {
    RT_TRY(rt_ctx_enter(ctx));
    if (!ev) return RT_OK;
    (void)hipEventDestroy(ev->ev);
    delete ev;
    return RT_OK;
}

extern "C" int32_t rt_mem_stats(rt_ctx* ctx, uint64_t* in_use, uint64_t* cached, uint64_t* device_allocs) {
    if (!ctx) return rt_fail(RT_E_INVALID, "null context");
    CtxGuard g(ctx);
    if (in_use) *in_use = ctx->bytes_in_use;
    if (cached) *cached = ctx->bytes_cached;
    if (device_allocs) *device_allocs = ctx->device_allocs;
    return RT_OK;
}

extern "C" int32_t rt_mem_trim(rt_ctx* ctx) {
    RT_TRY(rt_ctx_enter(ctx));
    CtxGuard g(ctx);
    RT_HIP(hipStreamSynchronize(ctx->stream));
    for (auto& kv : ctx->free_blocks) (void)hipFree(kv.second);
    ctx->free_blocks.clear();
    ctx->bytes_cached = 0;
    return RT_OK;
}
