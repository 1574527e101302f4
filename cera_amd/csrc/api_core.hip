// C ABI: context, device memory, events, weight upload and the kernel-level
// entry points (see include/cera_hip.h for the contract of each).
#include <cstring>
#include <new>

#include "attention.hip.h"
#include "gemv_launch.hip.h"
#include "gemv_nb.hip.h"
#include "glue.hip.h"
#include "cera_hip_kernels.h"
#include "host_common.h"
#include "quantize.hip.h"

bool cera_gemv_launch_q4k(const GemvArgs&, const GemvPlan&, int, bool, hipStream_t);
bool cera_gemv_launch_pair_q4k_q6k(const GemvPairArgs& a, const GemvPlan& pa, const GemvPlan& pb, hipStream_t s);
bool cera_gemv_nb_launch_q4k(const GemvNbArgs&, int, int, int, bool, uint32_t, hipStream_t);
bool cera_gemv_nb_launch_q6k(const GemvNbArgs&, int, int, int, bool, uint32_t, hipStream_t);
bool cera_gemv_nb_launch_q4_0(const GemvNbArgs&, int, int, int, bool, uint32_t, hipStream_t);
bool cera_gemv_nb_launch_q4_1(const GemvNbArgs&, int, int, int, bool, uint32_t, hipStream_t);
bool cera_gemv_nb_launch_q8_0(const GemvNbArgs&, int, int, int, bool, uint32_t, hipStream_t);
bool cera_gemv_launch_q6k(const GemvArgs&, const GemvPlan&, int, bool, hipStream_t);
bool cera_gemv_launch_q4_0(const GemvArgs&, const GemvPlan&, int, bool, hipStream_t);
bool cera_gemv_launch_q4_1(const GemvArgs&, const GemvPlan&, int, bool, hipStream_t);
bool cera_gemv_launch_q8_0(const GemvArgs&, const GemvPlan&, int, bool, hipStream_t);

// ---------------------------------------------------------------------------
// Fixed workspace of the allocation-free attention entry (cera_hip_attn_decode_dev_noalloc): the
// split-K partials of one decode-attention call.  The array's name is only a host-side handle;
// its device address is resolved once per device at context creation and that pointer is what
// kernels receive.  Every GPU holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[CERA_HIP_NOALLOC_WORKSPACE_BYTES];
static constexpr uint64_t NOALLOC_ML_BYTES = 128u << 10;   // (m, l) pairs in front, the accumulators behind
static constexpr int MAX_DEVICES = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[MAX_DEVICES] = {nullptr};

// with `device` current: the address of this device's copy of `scratch`
static hipError_t resolve_static_scratch(int device, void** out) {
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

static std::mutex g_err_mu;
static std::string g_err;

void cera_set_global_error(const std::string& s) {
    std::lock_guard<std::mutex> lk(g_err_mu);
    g_err = s;
}
cera_hip_status cera_fail(cera_hip_ctx* ctx, cera_hip_status st, const std::string& msg) {
    if (ctx) ctx->err = msg;
    cera_set_global_error(msg);
    return st;
}

bool cera_type_geometry(uint32_t t, uint32_t* e, uint32_t* b) {
    switch (t) {
        case CERA_HIP_F32: *e = 1; *b = 4; return true;
        case CERA_HIP_F16: case CERA_HIP_BF16: *e = 1; *b = 2; return true;
        case CERA_HIP_Q4_0: *e = 32; *b = 18; return true;
        case CERA_HIP_Q4_1: *e = 32; *b = 20; return true;
        case CERA_HIP_Q8_0: *e = 32; *b = 34; return true;
        case CERA_HIP_Q4_K: *e = 256; *b = 144; return true;
        case CERA_HIP_Q5_K: *e = 256; *b = 176; return true;
        case CERA_HIP_Q6_K: *e = 256; *b = 210; return true;
        default: return false;
    }
}

cera_hip_status cera_scratch(cera_hip_ctx* ctx, int slot, uint64_t nbytes, void** out) {
    if (nbytes == 0) nbytes = 256;
    if (ctx->scratch_bytes[slot] < nbytes) {
        if (ctx->scratch[slot]) {
            HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
            HIP_TRY(ctx, hipFree(ctx->scratch[slot]));
            ctx->scratch[slot] = nullptr;
            ctx->scratch_bytes[slot] = 0;
        }
        uint64_t want = (nbytes + 4095) & ~uint64_t(4095);
        HIP_TRY(ctx, hipMalloc(&ctx->scratch[slot], want));
        ctx->scratch_bytes[slot] = want;
    }
    *out = ctx->scratch[slot];
    return CERA_HIP_OK;
}

hipFunction_t cera_module_fn(cera_hip_ctx* ctx, const std::string& name) {
    if (!ctx->module) return nullptr;
    auto it = ctx->module_fns.find(name);
    if (it != ctx->module_fns.end()) return it->second;
    hipFunction_t f = nullptr;
    if (hipModuleGetFunction(&f, ctx->module, name.c_str()) != hipSuccess) {
        f = nullptr;
        (void)hipGetLastError();   // "not found" is an answer, not a sticky error
    }
    ctx->module_fns.emplace(name, f);
    return f;
}

cera_hip_status cera_module_launch(cera_hip_ctx* ctx, hipFunction_t f, uint32_t grid, uint32_t block, void* args) {
    void* params[] = {args};
    HIP_TRY(ctx, hipModuleLaunchKernel(f, grid, 1, 1, block, 1, 1, 0, ctx->stream, params, nullptr));
    return CERA_HIP_OK;
}

extern "C" {

cera_hip_status cera_hip_ctx_create(int device, const char* hsaco_path, cera_hip_ctx** out) {
    if (!out) return cera_fail(nullptr, CERA_HIP_ERR_ARGUMENT, "cera_hip_ctx_create: out is null");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0)
        return cera_fail(nullptr, CERA_HIP_ERR_DEVICE,
                         std::string("no HIP device available: ") + (e != hipSuccess ? hipGetErrorString(e) : "count is 0"));
    if (device < 0 || device >= n || device >= MAX_DEVICES) return cera_fail(nullptr, CERA_HIP_ERR_ARGUMENT, "device index out of range");
    cera_hip_ctx* ctx = new (std::nothrow) cera_hip_ctx();
    if (!ctx) return cera_fail(nullptr, CERA_HIP_ERR_OOM, "host allocation failed");
    ctx->device = device;
    hipDeviceProp_t prop;
    if ((e = hipSetDevice(device)) != hipSuccess || (e = hipGetDeviceProperties(&prop, device)) != hipSuccess ||
        (e = resolve_static_scratch(device, &ctx->static_scratch)) != hipSuccess ||
        (e = hipStreamCreate(&ctx->stream)) != hipSuccess) {
        delete ctx;
        return cera_fail(nullptr, CERA_HIP_ERR_DEVICE, std::string("device init: ") + hipGetErrorString(e));
    }
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        std::string arch = prop.gcnArchName;
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return cera_fail(nullptr, CERA_HIP_ERR_DEVICE, "kernels are built for gfx950 only; device is " + arch);
    }
    ctx->n_cu = static_cast<uint32_t>(prop.multiProcessorCount);
    if (hsaco_path) {
        if ((e = hipModuleLoad(&ctx->module, hsaco_path)) != hipSuccess) {
            (void)hipGetLastError();   // the failed load must not surface as a later call's error
            (void)hipStreamDestroy(ctx->stream);
            delete ctx;
            return cera_fail(nullptr, CERA_HIP_ERR_DEVICE, std::string("hipModuleLoad(") + hsaco_path + "): " + hipGetErrorString(e));
        }
        if (!cera_module_fn(ctx, "cera_k_quantize_q8_0")) {
            (void)hipModuleUnload(ctx->module);
            (void)hipStreamDestroy(ctx->stream);
            delete ctx;
            return cera_fail(nullptr, CERA_HIP_ERR_ARGUMENT, std::string(hsaco_path) + " is not this library's code object (no cera_k_quantize_q8_0)");
        }
    }
    *out = ctx;
    return CERA_HIP_OK;
}

void cera_hip_ctx_destroy(cera_hip_ctx* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto& p : ctx->scratch)
        if (p) (void)hipFree(p);
    if (ctx->attn_acc) (void)hipFree(ctx->attn_acc);
    if (ctx->attn_ml) (void)hipFree(ctx->attn_ml);
    for (int i = 0; i < 2; ++i) {
        if (ctx->pin[i]) (void)hipHostFree(ctx->pin[i]);
        if (ctx->pin_ev[i]) (void)hipEventDestroy(ctx->pin_ev[i]);
    }
    if (ctx->word_host) (void)hipHostFree(ctx->word_host);
    if (ctx->module) (void)hipModuleUnload(ctx->module);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

const char* cera_hip_last_error(const cera_hip_ctx* ctx) {
    if (ctx) return ctx->err.c_str();
    static thread_local std::string copy;
    std::lock_guard<std::mutex> lk(g_err_mu);
    copy = g_err;
    return copy.c_str();
}

cera_hip_status cera_hip_sync(cera_hip_ctx* ctx) {
    if (!ctx) return CERA_HIP_ERR_ARGUMENT;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return CERA_HIP_OK;
}

cera_hip_status cera_hip_ctx_set_decode_copies(cera_hip_ctx* ctx, int enabled) {
    if (!ctx) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    ctx->decode_copies = enabled != 0;
    return CERA_HIP_OK;
}

cera_hip_status cera_hip_device_info(cera_hip_ctx* ctx, char* name256, uint32_t* n_cu, uint64_t* hbm) {
    if (!ctx) return CERA_HIP_ERR_ARGUMENT;
    hipDeviceProp_t prop;
    HIP_TRY(ctx, hipGetDeviceProperties(&prop, ctx->device));
    if (name256) {
        std::snprintf(name256, 256, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (n_cu) *n_cu = static_cast<uint32_t>(prop.multiProcessorCount);
    if (hbm) *hbm = prop.totalGlobalMem;
    return CERA_HIP_OK;
}

// ---- memory / events --------------------------------------------------------
cera_hip_status cera_hip_malloc(cera_hip_ctx* ctx, uint64_t nbytes, void** out) {
    if (!ctx || !out) return CERA_HIP_ERR_ARGUMENT;
    *out = nullptr;
    HIP_TRY(ctx, hipMalloc(out, nbytes ? nbytes : 256));
    return CERA_HIP_OK;
}
cera_hip_status cera_hip_free(cera_hip_ctx* ctx, void* dev) {
    if (!ctx) return CERA_HIP_ERR_ARGUMENT;
    if (!dev) return CERA_HIP_OK;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    HIP_TRY(ctx, hipFree(dev));
    return CERA_HIP_OK;
}
cera_hip_status cera_hip_upload(cera_hip_ctx* ctx, void* dst, const void* src, uint64_t n) {
    if (!ctx || (!dst && n) || (!src && n)) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0) return CERA_HIP_OK;
    HIP_TRY(ctx, hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return CERA_HIP_OK;
}
// Device -> pageable host memory.  The runtime's own route for a pageable destination moves
// copies of up to a few MB at about 2 GB/s (0.26 ms for one row of logits) and large ones at
// 17 GB/s (it pins the destination).  Staged through two pinned chunks, the DMA of chunk i+1
// running while the CPU copies chunk i out, the same copies take 0.06 ms and run at 25 GB/s;
// only beyond PIN_DIRECT bytes is the runtime's route taken.
static constexpr uint64_t PIN_CHUNK = 1u << 20, PIN_DIRECT = 256u << 20;
cera_hip_status cera_hip_download(cera_hip_ctx* ctx, void* dst, const void* src, uint64_t n) {
    if (!ctx || (!dst && n) || (!src && n)) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0) return CERA_HIP_OK;
    if (n >= PIN_DIRECT) {
        HIP_TRY(ctx, hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        return CERA_HIP_OK;
    }
    std::lock_guard<std::mutex> lk(ctx->pin_mu);
    for (int i = 0; i < 2; ++i) {
        if (!ctx->pin[i]) HIP_TRY(ctx, hipHostMalloc(&ctx->pin[i], PIN_CHUNK, hipHostMallocDefault));
        if (!ctx->pin_ev[i]) HIP_TRY(ctx, hipEventCreateWithFlags(&ctx->pin_ev[i], hipEventDisableTiming));
    }
    const uint64_t n_chunks = (n + PIN_CHUNK - 1) / PIN_CHUNK;
    for (uint64_t i = 0; i <= n_chunks; ++i) {
        if (i < n_chunks) {   // chunk i-2, the last user of this pinned buffer, was copied out one turn ago
            const uint64_t off = i * PIN_CHUNK, len = std::min(PIN_CHUNK, n - off);
            HIP_TRY(ctx, hipMemcpyAsync(ctx->pin[i & 1], static_cast<const char*>(src) + off, len, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, hipEventRecord(ctx->pin_ev[i & 1], ctx->stream));
        }
        if (i >= 1) {
            const uint64_t j = i - 1, off = j * PIN_CHUNK, len = std::min(PIN_CHUNK, n - off);
            HIP_TRY(ctx, hipEventSynchronize(ctx->pin_ev[j & 1]));
            std::memcpy(static_cast<char*>(dst) + off, ctx->pin[j & 1], len);
        }
    }
    return CERA_HIP_OK;
}
cera_hip_status cera_hip_copy_dev(cera_hip_ctx* ctx, void* dst, const void* src, uint64_t n) {
    if (!ctx || (!dst && n) || (!src && n)) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0) return CERA_HIP_OK;
    HIP_TRY(ctx, hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, ctx->stream));
    return CERA_HIP_OK;
}
// Plain streaming copy, 16 bytes per lane per step: a kernel of exactly known HBM traffic
// (n read + n written) against which hardware byte counters can be calibrated.
static __global__ void __launch_bounds__(256) copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, uint64_t n16) {
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += uint64_t(gridDim.x) * blockDim.x)
        dst[i] = src[i];
}
cera_hip_status cera_hip_copy_kernel(cera_hip_ctx* ctx, void* dst, const void* src, uint64_t n) {
    if (!ctx || !dst || !src) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0 || n % 16 || (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "copy_kernel: size and pointers must be multiples of 16 bytes");
    uint64_t n16 = n / 16;
    uint32_t blocks = static_cast<uint32_t>(std::min<uint64_t>((n16 + 255) / 256, uint64_t(ctx->n_cu) * 16));
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, ctx->stream, static_cast<uint4*>(dst),
                       static_cast<const uint4*>(src), n16);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}
cera_hip_status cera_hip_event_create(cera_hip_ctx* ctx, cera_hip_event** out) {
    if (!ctx || !out) return CERA_HIP_ERR_ARGUMENT;
    cera_hip_event* e = new (std::nothrow) cera_hip_event();
    if (!e) return cera_fail(ctx, CERA_HIP_ERR_OOM, "host allocation failed");
    hipError_t r = hipEventCreate(&e->ev);
    if (r != hipSuccess) {
        delete e;
        return cera_fail(ctx, CERA_HIP_ERR_DEVICE, std::string("hipEventCreate: ") + hipGetErrorString(r));
    }
    *out = e;
    return CERA_HIP_OK;
}
void cera_hip_event_destroy(cera_hip_event* e) {
    if (!e) return;
    (void)hipEventDestroy(e->ev);
    delete e;
}
cera_hip_status cera_hip_event_record(cera_hip_ctx* ctx, cera_hip_event* e) {
    if (!ctx || !e) return CERA_HIP_ERR_ARGUMENT;
    HIP_TRY(ctx, hipEventRecord(e->ev, ctx->stream));
    return CERA_HIP_OK;
}
cera_hip_status cera_hip_event_elapsed_ms(cera_hip_ctx* ctx, cera_hip_event* a, cera_hip_event* b, float* ms) {
    if (!ctx || !a || !b || !ms) return CERA_HIP_ERR_ARGUMENT;
    HIP_TRY(ctx, hipEventSynchronize(b->ev));
    HIP_TRY(ctx, hipEventElapsedTime(ms, a->ev, b->ev));
    return CERA_HIP_OK;
}

// ---- weights ------------------------------------------------------------------
static cera_hip_status check_tensor(cera_hip_ctx* ctx, const cera_hip_tensor* t, uint64_t* row_bytes) {
    if (!t || !t->data) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "tensor or tensor data is null");
    uint32_t e, b;
    if (!cera_type_geometry(t->ggml_type, &e, &b))
        return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                         "no hip kernel for ggml type " + std::to_string(t->ggml_type));
    if (t->m == 0 || t->k == 0 || t->k % e)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "k=" + std::to_string(t->k) + " is not a whole number of " +
                                                      std::to_string(e) + "-element blocks (or m/k is zero)");
    *row_bytes = t->k / e * b;
    if (t->nbytes != t->m * *row_bytes)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "tensor nbytes " + std::to_string(t->nbytes) + " != m*row_bytes " +
                                                      std::to_string(t->m * *row_bytes));
    if (t->m > 0xFFFFFFFFull || t->k > 0xFFFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "dimension exceeds 2^32");
    return CERA_HIP_OK;
}

static cera_hip_status alloc_dtensor(cera_hip_ctx* ctx, uint32_t dtype, uint64_t m, uint64_t k, uint64_t row_bytes,
                                     cera_hip_dtensor** out) {
    cera_hip_dtensor* d = new (std::nothrow) cera_hip_dtensor();
    if (!d) return cera_fail(ctx, CERA_HIP_ERR_OOM, "host allocation failed");
    d->dtype = dtype; d->m = m; d->k = k; d->row_bytes = row_bytes; d->nbytes = m * row_bytes;
    // 64 bytes of slack: a dead lane may read up to one unit past its own data
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&d->dev), d->nbytes + 64);
    if (e != hipSuccess) {
        delete d;
        return cera_fail(ctx, e == hipErrorOutOfMemory ? CERA_HIP_ERR_OOM : CERA_HIP_ERR_DEVICE,
                         std::string("hipMalloc(weights): ") + hipGetErrorString(e));
    }
    *out = d;
    return CERA_HIP_OK;
}

cera_hip_status cera_hip_tensor_upload(cera_hip_ctx* ctx, const cera_hip_tensor* t, cera_hip_dtensor** out) {
    if (!ctx || !out) return CERA_HIP_ERR_ARGUMENT;
    *out = nullptr;
    uint64_t rb;
    CERA_TRY(check_tensor(ctx, t, &rb));
    cera_hip_dtensor* d;
    CERA_TRY(alloc_dtensor(ctx, t->ggml_type, t->m, t->k, rb, &d));
    hipError_t e = hipMemcpyAsync(d->dev, t->data, d->nbytes, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(d->dev);
        delete d;
        return cera_fail(ctx, CERA_HIP_ERR_DEVICE, std::string("weight upload: ") + hipGetErrorString(e));
    }
    *out = d;
    return CERA_HIP_OK;
}

cera_hip_status cera_hip_tensor_clone(cera_hip_ctx* ctx, const cera_hip_dtensor* src, cera_hip_dtensor** out) {
    if (!ctx || !src || !out) return CERA_HIP_ERR_ARGUMENT;
    *out = nullptr;
    cera_hip_dtensor* d;
    CERA_TRY(alloc_dtensor(ctx, src->dtype, src->m, src->k, src->row_bytes, &d));
    hipError_t e = hipMemcpyAsync(d->dev, src->dev, d->nbytes, hipMemcpyDeviceToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(d->dev);
        delete d;
        return cera_fail(ctx, CERA_HIP_ERR_DEVICE, std::string("weight clone: ") + hipGetErrorString(e));
    }
    *out = d;
    return CERA_HIP_OK;
}

void cera_hip_tensor_free(cera_hip_ctx* ctx, cera_hip_dtensor* d) {
    if (!d) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (d->dev && d->owns) (void)hipFree(d->dev);
    if (d->dev_stream) (void)hipFree(d->dev_stream);
    delete d;
}
uint64_t cera_hip_tensor_nbytes(const cera_hip_dtensor* d) { return d ? d->nbytes : 0; }

}  // extern "C"

cera_hip_status cera_tensor_upload_concat(cera_hip_ctx* ctx, const cera_hip_tensor* const* parts, int n_parts,
                                          cera_hip_dtensor** fused, cera_hip_dtensor** views) {
    *fused = nullptr;
    uint64_t rb = 0, rows = 0;
    for (int i = 0; i < n_parts; ++i) {
        uint64_t r;
        CERA_TRY(check_tensor(ctx, parts[i], &r));
        if (parts[i]->ggml_type != parts[0]->ggml_type || parts[i]->k != parts[0]->k)
            return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "concat: parts differ in type or k");
        rb = r;
        rows += parts[i]->m;
    }
    cera_hip_dtensor* f;
    CERA_TRY(alloc_dtensor(ctx, parts[0]->ggml_type, rows, parts[0]->k, rb, &f));
    uint64_t off = 0;
    for (int i = 0; i < n_parts; ++i) {
        hipError_t e = hipMemcpyAsync(f->dev + off, parts[i]->data, parts[i]->nbytes, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        cera_hip_dtensor* v = e == hipSuccess ? new (std::nothrow) cera_hip_dtensor() : nullptr;
        if (!v) {
            for (int j = 0; j < i; ++j) { delete views[j]; views[j] = nullptr; }
            cera_hip_tensor_free(ctx, f);
            return cera_fail(ctx, e != hipSuccess ? CERA_HIP_ERR_DEVICE : CERA_HIP_ERR_OOM,
                             e != hipSuccess ? std::string("weight upload: ") + hipGetErrorString(e) : "host allocation failed");
        }
        v->dtype = f->dtype; v->m = parts[i]->m; v->k = f->k; v->row_bytes = rb; v->nbytes = parts[i]->nbytes;
        v->dev = f->dev + off; v->owns = false;
        views[i] = v;
        off += parts[i]->nbytes;
    }
    *fused = f;
    return CERA_HIP_OK;
}

// ---------------------------------------------------------------------------
// launchers
cera_hip_status cera_launch_quantize(cera_hip_ctx* ctx, const float* x, uint64_t k, float* scales, int8_t* quants,
                                     float* bsum) {
    if (k == 0 || k % 32) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "quantize_q8_0: k must be a positive multiple of 32");
    uint64_t threads = k / 4;
    dim3 grid(static_cast<uint32_t>((threads + 255) / 256));
    if (hipFunction_t f = cera_module_fn(ctx, "cera_k_quantize_q8_0")) {
        cera_k_quantize_q8_0_args a{x, k, scales, quants, bsum};
        return cera_module_launch(ctx, f, grid.x, 256, &a);
    }
    hipLaunchKernelGGL(quantize_q8_0_kernel, grid, dim3(256), 0, ctx->stream, x, k, scales, quants, bsum);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

// weights per lane unit of the decode GEMV kernels
static uint32_t cera_gemv_unit_elems(uint32_t dtype) { return (dtype == CERA_HIP_Q6_K || dtype == CERA_HIP_Q4_K) ? 64 : 32; }

static bool is_int8_type(uint32_t t) {
    return t == CERA_HIP_Q4_0 || t == CERA_HIP_Q4_1 || t == CERA_HIP_Q8_0 || t == CERA_HIP_Q4_K || t == CERA_HIP_Q6_K;
}

cera_hip_status cera_launch_gemv(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const cera_hip_dtensor* w2,
                                 const float* xs, const int8_t* xq, float* y, const float* resid, int epi,
                                 int32_t* dbg_dots, int32_t* dbg_asums) {
    if (!is_int8_type(w->dtype))
        return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "no int8 gemv kernel for ggml type " + std::to_string(w->dtype));
    if (epi == CERA_EPI_SILU_MUL) {
        if (!w2 || w2->dtype != w->dtype || w2->m != w->m || w2->k != w->k)
            return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "fused gate/up gemv needs two matrices of identical type and shape");
    }
    if (epi == CERA_EPI_ADD && !resid) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "residual pointer is null");
    // unit = 32 weights, except the K-quants whose lanes take 64
    uint32_t n_units = static_cast<uint32_t>(w->k / cera_gemv_unit_elems(w->dtype));
    GemvArgs a;
    a.w = w->dev;
    a.w2 = w2 ? w2->dev : nullptr;
    a.xq = xq;
    a.xs = xs;
    a.y = y;
    a.resid = resid;
    a.m = static_cast<uint32_t>(w->m);
    a.n_units = n_units;
    a.row_bytes = static_cast<uint32_t>(w->row_bytes);
    a.dbg_dots = dbg_dots;
    a.dbg_asums = dbg_asums;
    a.dbg_stride = static_cast<uint32_t>(w->dtype == CERA_HIP_Q6_K ? w->k / 16 : w->k / 32);
    const bool dbg = dbg_dots != nullptr;
    GemvPlan p;
    // rows in flight: a K-quant row unit is 12-15 registers (two matrices in the fused pair)
    const int max_rb = w->dtype == CERA_HIP_Q4_K ? (epi == CERA_EPI_SILU_MUL ? 1 : 2) : (w->dtype == CERA_HIP_Q6_K ? 2 : 4);
    if (!gemv_plan(a.m, n_units, ctx->n_cu, dbg, max_rb, &p, epi == CERA_EPI_SILU_MUL))
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemv: k=" + std::to_string(w->k) + " exceeds the 32768 supported by the register-resident kernel");
    a.rows_per_wave = p.rows_per_block;
    // with a loaded code object, the instances it exports (one unit per lane, K split 1/2/4/8, two
    // rows in flight, store / add epilogue) are launched from it; everything else is embedded
    if (ctx->module && !dbg && p.U == 1 && p.KS != 7 && epi != CERA_EPI_SILU_MUL) {
        static const char* const tn[] = {"q4_0", "q4_1", "q8_0", "q4_k", "q6_k"};
        const int ti = w->dtype == CERA_HIP_Q4_0 ? 0 : w->dtype == CERA_HIP_Q4_1 ? 1 : w->dtype == CERA_HIP_Q8_0 ? 2 : w->dtype == CERA_HIP_Q4_K ? 3 : 4;
        const std::string name = std::string("cera_k_gemv_") + tn[ti] + "_ks" + std::to_string(p.KS) + (epi == CERA_EPI_ADD ? "_add" : "_store");
        if (hipFunction_t f = cera_module_fn(ctx, name)) {
            a.rows_per_wave = (p.rows_per_block + 1) / 2 * 2;
            const uint32_t n_blocks = (a.m + a.rows_per_wave - 1) / a.rows_per_wave;
            return cera_module_launch(ctx, f, n_blocks, 64 * p.KS, &a);
        }
    }
    bool ok = false;
    switch (w->dtype) {
        case CERA_HIP_Q4_K: ok = cera_gemv_launch_q4k(a, p, epi, dbg, ctx->stream); break;
        case CERA_HIP_Q6_K: ok = cera_gemv_launch_q6k(a, p, epi, dbg, ctx->stream); break;
        case CERA_HIP_Q4_0: ok = cera_gemv_launch_q4_0(a, p, epi, dbg, ctx->stream); break;
        case CERA_HIP_Q4_1: ok = cera_gemv_launch_q4_1(a, p, epi, dbg, ctx->stream); break;
        case CERA_HIP_Q8_0: ok = cera_gemv_launch_q8_0(a, p, epi, dbg, ctx->stream); break;
    }
    if (!ok) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemv: no kernel instance for this shape");
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

// A short batch of tokens through one matrix with the weights streamed once per 8 tokens:
// y[t][row] (row stride 1, token stride y_stride) = W . x_t (+ resid, same layout).  *launched is
// false when the shape has no multi-token instance (two units per lane, i.e. very long rows):
// the caller then takes the GEMM route.
cera_hip_status cera_launch_gemv_nb(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                    uint32_t xs_stride, uint32_t xq_stride, uint32_t n_tok, float* y, uint32_t y_stride,
                                    const float* resid, bool* launched) {
    *launched = false;
    if (!is_int8_type(w->dtype) || n_tok == 0) return CERA_HIP_OK;
    // a decode copy and rows of one pass per lane: the streaming row kernel (same bits)
    CERA_TRY(cera_launch_row_gemv_nb(ctx, w, xs, xq, xs_stride, xq_stride, n_tok, y, y_stride, resid, launched));
    if (*launched) return CERA_HIP_OK;
    const uint32_t n_units = static_cast<uint32_t>(w->k / cera_gemv_unit_elems(w->dtype));
    GemvPlan p;
    if (!gemv_plan(static_cast<uint32_t>(w->m), n_units, ctx->n_cu, false, 2, &p) || p.U != 1) return CERA_HIP_OK;
    const int KS = p.KS == 7 ? 8 : p.KS;   // instantiated widths: 1, 2, 4, 8 (surplus lanes carry zero activations)
    GemvNbArgs a;
    a.w = w->dev;
    a.m = static_cast<uint32_t>(w->m);
    a.n_units = n_units;
    a.row_bytes = static_cast<uint32_t>(w->row_bytes);
    a.rows_per_block = p.rows_per_block;
    a.xq_stride = xq_stride;
    a.xs_stride = xs_stride;
    a.y_stride = y_stride;
    for (uint32_t t0 = 0; t0 < n_tok; t0 += 8) {
        const uint32_t nt = std::min(8u, n_tok - t0);
        const int NB = nt <= 2 ? 2 : (nt <= 4 ? 4 : 8);
        a.n_tok = nt;
        a.xq = xq + static_cast<uint64_t>(t0) * xq_stride;
        a.xs = xs + static_cast<uint64_t>(t0) * xs_stride;
        a.y = y + static_cast<uint64_t>(t0) * y_stride;
        a.resid = resid ? resid + static_cast<uint64_t>(t0) * y_stride : nullptr;
        bool ok = false;
        switch (w->dtype) {
            case CERA_HIP_Q4_K: ok = cera_gemv_nb_launch_q4k(a, KS, p.RB, NB, resid != nullptr, p.n_blocks, ctx->stream); break;
            case CERA_HIP_Q6_K: ok = cera_gemv_nb_launch_q6k(a, KS, p.RB, NB, resid != nullptr, p.n_blocks, ctx->stream); break;
            case CERA_HIP_Q4_0: ok = cera_gemv_nb_launch_q4_0(a, KS, p.RB, NB, resid != nullptr, p.n_blocks, ctx->stream); break;
            case CERA_HIP_Q4_1: ok = cera_gemv_nb_launch_q4_1(a, KS, p.RB, NB, resid != nullptr, p.n_blocks, ctx->stream); break;
            case CERA_HIP_Q8_0: ok = cera_gemv_nb_launch_q8_0(a, KS, p.RB, NB, resid != nullptr, p.n_blocks, ctx->stream); break;
        }
        if (!ok) return t0 == 0 ? CERA_HIP_OK : cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemv_nb: no kernel instance for this shape");
        HIP_TRY(ctx, hipGetLastError());
    }
    *launched = true;
    return CERA_HIP_OK;
}

// Two projections of the same quantized activations in one launch (plain store epilogue).
// *launched is false when no paired kernel instance covers the two shapes: the caller then
// launches them one after the other.
cera_hip_status cera_launch_gemv_pair(cera_hip_ctx* ctx, const cera_hip_dtensor* wa, const cera_hip_dtensor* wb,
                                      const float* xs, const int8_t* xq, float* ya, float* yb, bool* launched) {
    *launched = false;
    if (wa->dtype != CERA_HIP_Q4_K || wb->dtype != CERA_HIP_Q6_K || wa->k != wb->k) return CERA_HIP_OK;
    auto fill = [&](const cera_hip_dtensor* w, float* y, uint32_t n_units, GemvArgs* a) {
        a->w = w->dev; a->w2 = nullptr; a->xq = xq; a->xs = xs; a->y = y; a->resid = nullptr;
        a->m = static_cast<uint32_t>(w->m); a->n_units = n_units; a->row_bytes = static_cast<uint32_t>(w->row_bytes);
        a->dbg_dots = nullptr; a->dbg_asums = nullptr; a->dbg_stride = 0;
    };
    GemvPairArgs p;
    GemvPlan pa, pb;
    const uint32_t ua = static_cast<uint32_t>(wa->k / Q4K::ELEMS_PER_UNIT), ub = static_cast<uint32_t>(wb->k / Q6K::ELEMS_PER_UNIT);
    if (!gemv_plan(static_cast<uint32_t>(wa->m), ua, ctx->n_cu, false, 2, &pa)) return CERA_HIP_OK;
    if (!gemv_plan(static_cast<uint32_t>(wb->m), ub, ctx->n_cu, false, 2, &pb)) return CERA_HIP_OK;
    fill(wa, ya, ua, &p.a);
    fill(wb, yb, ub, &p.b);
    p.a.rows_per_wave = pa.rows_per_block;
    p.b.rows_per_wave = pb.rows_per_block;
    p.n_blocks_a = pa.n_blocks;
    if (!cera_gemv_launch_pair_q4k_q6k(p, pa, pb, ctx->stream)) return CERA_HIP_OK;
    HIP_TRY(ctx, hipGetLastError());
    *launched = true;
    return CERA_HIP_OK;
}

cera_hip_status cera_pinned_word(cera_hip_ctx* ctx, uint32_t** host, uint32_t** dev) {
    if (!ctx->word_host) {
        void *h = nullptr, *d = nullptr;
        HIP_TRY(ctx, hipHostMalloc(&h, 64, hipHostMallocMapped));
        const hipError_t e = hipHostGetDevicePointer(&d, h, 0);
        if (e != hipSuccess) {
            (void)hipHostFree(h);
            return cera_fail(ctx, CERA_HIP_ERR_DEVICE, std::string("hipHostGetDevicePointer: ") + hipGetErrorString(e));
        }
        ctx->word_host = static_cast<uint32_t*>(h);
        ctx->word_dev = static_cast<uint32_t*>(d);
    }
    *host = ctx->word_host;
    *dev = ctx->word_dev;
    return CERA_HIP_OK;
}

cera_hip_status cera_launch_argmax(cera_hip_ctx* ctx, const float* x, uint32_t n, uint32_t* out_dev, uint32_t* out_host_mapped) {
    void* part;
    CERA_TRY(cera_scratch(ctx, 8, ARGMAX_PARTS * 8, &part));
    float* pv = static_cast<float*>(part);
    uint32_t* pi = reinterpret_cast<uint32_t*>(pv + ARGMAX_PARTS);
    const uint32_t np = std::max(1u, std::min<uint32_t>(ARGMAX_PARTS, (n + 1023) / 1024));
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(np), dim3(256), 0, ctx->stream, x, n, pv, pi);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, ctx->stream, pv, pi, np, out_dev, out_host_mapped);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

struct AttnLaunch {
    const float* q;
    uint32_t seq_len, max_seq;
    float scale;
    uint32_t n_heads, n_kv_heads, n_queries, q_stride, G, S, n_parts, part_keys, chunks_per_part;
    uint32_t Gw;   // query heads one decode wavefront serves (divides G); G / Gw wavefronts share a kv head's rows
    bool batch, fused_new_kv;
    AttnNewKV nk;
    float *acc, *ml;   // split-K partials: (o) and (m, l) per (query, head, part)
};

// G = heads per wavefront; a.G = heads per kv head (G or 2 G)
template <int G, typename KV, int HD>
static void attn_launch_decode_g(cera_hip_ctx* ctx, const AttnLaunch& a, const KV* kc, const KV* vc) {
    // a workgroup is four wavefronts = four consecutive parts of one (kv head, sub-group, query);
    // the kernel maps launch indices to them XCD by XCD, so the count is rounded up to whole eights
    const uint32_t groups = (a.n_parts + 3) / 4 * a.n_kv_heads, reps = (a.G / G) * a.n_queries;
    const dim3 grid((groups + 7) / 8 * 8 * reps), block(256);
    // one query and one wavefront per kv head and key range: every K/V row is read exactly once,
    // which is what the non-temporal instances want (long chunks only: short ones prefetch V
    // with K and are latency-bound)
    const bool nt = a.G == G && a.n_queries == 1 && a.S >= 4;
#define ATTN_LAUNCH_SN(SS, NT)                                                                                       \
    do {                                                                                                             \
        if (a.fused_new_kv)                                                                                          \
            hipLaunchKernelGGL((attn_decode_partial_kernel<G, SS, true, KV, HD, NT>), grid, block, 0, ctx->stream, a.q,  \
                               kc, vc, a.seq_len, a.max_seq, a.scale, a.chunks_per_part, a.n_parts, a.q_stride, a.G, \
                               a.n_kv_heads, a.n_queries, a.acc, a.ml, a.nk);                                        \
        else                                                                                                         \
            hipLaunchKernelGGL((attn_decode_partial_kernel<G, SS, false, KV, HD, NT>), grid, block, 0, ctx->stream, a.q, \
                               kc, vc, a.seq_len, a.max_seq, a.scale, a.chunks_per_part, a.n_parts, a.q_stride, a.G, \
                               a.n_kv_heads, a.n_queries, a.acc, a.ml, a.nk);                                        \
    } while (0)
#define ATTN_LAUNCH_S(SS) ATTN_LAUNCH_SN(SS, false)
    switch (a.S) {
        case 1: ATTN_LAUNCH_S(1); break;
        case 2: ATTN_LAUNCH_S(2); break;
        case 4:
            if (nt) ATTN_LAUNCH_SN(4, true);
            else ATTN_LAUNCH_S(4);
            break;
        default:
            if (nt) ATTN_LAUNCH_SN(8, true);
            else ATTN_LAUNCH_S(8);
            break;
    }
#undef ATTN_LAUNCH_SN
#undef ATTN_LAUNCH_S
}

template <typename KV, int HD>
static void attn_launch_partials(cera_hip_ctx* ctx, const AttnLaunch& a, const KV* kc, const KV* vc) {
    if (a.batch) {
        // heaviest query blocks (most visible keys) first
        const dim3 pgrid((a.n_queries + 31) / 32, a.n_kv_heads, a.n_parts);
#define ATTN_PF(GG)                                                                                                        \
    hipLaunchKernelGGL((attn_prefill_partial_kernel<KV, HD, GG>), pgrid, dim3(64 * GG), 0, ctx->stream, a.q, kc, vc, a.seq_len, \
                       a.n_queries, a.max_seq, a.scale, a.part_keys, a.n_parts, a.q_stride, a.acc, a.ml)
        switch (a.G) {   // any group of up to eight heads: one wavefront per head, 64 G threads
            case 1: ATTN_PF(1); break;
            case 2: ATTN_PF(2); break;
            case 3: ATTN_PF(3); break;
            case 4: ATTN_PF(4); break;
            case 5: ATTN_PF(5); break;
            case 6: ATTN_PF(6); break;
            case 7: ATTN_PF(7); break;
            default: ATTN_PF(8); break;
        }
#undef ATTN_PF
        return;
    }
    // A wavefront's time is largely its own instruction stream, which grows with the heads it
    // serves, so groups of 4 and 8 heads are split over two wavefronts (the K/V rows both read come
    // from cache the second time: the kernel places them on one XCD): 580 -> 590 tok/s on the 8B
    // model at ~640 keys, 5-15 % per call from 1k to 16k keys.  One head per wavefront gains nothing
    // over two.  From 16k keys on an f32 cache is bound by bytes: a group keeps one wavefront, every
    // K/V row is then read exactly once and the loads carry the non-temporal hint (131072 keys:
    // 5.50 TB/s split, 5.85 unsplit, 6.42 unsplit and non-temporal; 16384 keys: the same time either
    // way).  An f16 cache moves half the bytes for the same arithmetic and keeps the split up to 32k
    // keys (20000 keys: 30.4 -> 24.3 us; 65536: 58.4 unsplit, 62.0 split).  Groups of 8 heads do
    // twice the arithmetic per K/V byte and are never bound by bytes: they keep the split at every
    // length (64 / 8 heads, 131072 keys: 279.5 -> 207.3 us; f16 cache, 32768 keys: 91.0 -> 54.5).
    // Group sizes that are not powers of two (Qwen2's 28 / 4 and 12 / 2 heads) run the widest
    // instance that divides them -- seven one-head wavefronts, three two-head ones -- sharing the
    // kv head's rows the same way.
    switch (a.Gw) {
        case 1: attn_launch_decode_g<1, KV, HD>(ctx, a, kc, vc); break;
        case 2: attn_launch_decode_g<2, KV, HD>(ctx, a, kc, vc); break;
        case 4: attn_launch_decode_g<4, KV, HD>(ctx, a, kc, vc); break;
        default: attn_launch_decode_g<8, KV, HD>(ctx, a, kc, vc); break;
    }
}

cera_hip_status cera_launch_attn(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc,
                                 uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                 uint64_t max_seq, float scale, uint32_t n_splits, uint32_t n_queries, float* out,
                                 float* out_scales, int8_t* out_quants, float* out_bsum, const AttnNewKV* new_kv,
                                 bool kv_f16, const AttnWorkspace* ws) {
    if (n_kv_heads == 0 || n_heads % n_kv_heads) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attention: n_heads must be a multiple of n_kv_heads");
    if (n_queries == 0 || n_queries > 65535) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attention: 1..65535 queries per call");
    if (!cera_attn_shape_tuned(n_heads, n_kv_heads, head_dim)) {
        // Any other head size (a multiple of 8 up to 256) or group size, as decode_attention takes them
        // (cera/src/model/transformer.rs:1249-1305): one launch of the generic kernel per query, then the
        // Q8_0 quantization of the outputs.  Correct and slow; no model of the benchmark configs comes here.
        if (head_dim % 8 || head_dim > 256 || head_dim == 0)
            return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attention: head_dim must be a multiple of 8, at most 256");
        if (new_kv) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "attention: fused RoPE/append needs head_dim 64 or 128 and at most 8 heads per kv head");
        if (seq_len == 0 || seq_len + n_queries - 1 > max_seq || max_seq > 0x7FFFFFFFull)
            return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attention: need 0 < seq_len <= max_seq < 2^31");
        void* scores;
        CERA_TRY(cera_scratch(ctx, 13, static_cast<uint64_t>(n_heads) * max_seq * sizeof(float), &scores));
        const uint64_t q_dim = static_cast<uint64_t>(n_heads) * head_dim;
        for (uint32_t i = 0; i < n_queries; ++i)
            CERA_TRY(cera_launch_attn_generic(ctx, q + i * q_dim, kc, vc, n_heads, n_kv_heads, head_dim,
                                              static_cast<uint32_t>(seq_len) + i, static_cast<uint32_t>(max_seq), scale,
                                              static_cast<float*>(scores), out + i * q_dim, kv_f16));
        if (out_quants) {
            if (q_dim % 32) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attention: n_heads * head_dim must be a multiple of 32 to quantize the output");
            CERA_TRY(cera_launch_quantize(ctx, out, q_dim * n_queries, out_scales, out_quants, out_bsum));
        }
        return CERA_HIP_OK;
    }
    uint32_t G = n_heads / n_kv_heads;
    // seq_len = keys visible to the first query; the last query sees seq_len + n_queries - 1
    const uint64_t last_len = seq_len + n_queries - 1;
    if (seq_len == 0 || last_len > max_seq || max_seq > 0x7FFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attention: need 0 < seq_len <= max_seq < 2^31");
    // A batch of queries (prefill) runs the tiled MFMA kernel: a K/V tile is read once per 32
    // queries instead of once per query.  Parts of 128 keys while the context is short, about
    // eight parts per query block beyond that.
    if (new_kv && n_queries != 1) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "attention: fused RoPE/append is for single-token decode");
    const bool batch = n_queries >= 16;
    if (batch && (reinterpret_cast<uintptr_t>(q) & 15)) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "attention: a query batch must be 16-byte aligned");
    const AttnNewKV nk = new_kv ? *new_kv : AttnNewKV{};
    uint32_t n_parts, part_keys = 0, chunks_per_part = 0;
    uint32_t S = 1;
    uint32_t Gw = G;   // decode: heads per wavefront
    if (batch) {
        const uint64_t want = n_queries >= 1024 ? 4 : 8;   // many query blocks fill the chip with fewer parts
        part_keys = last_len <= 1024 ? 128u : static_cast<uint32_t>(((last_len + want - 1) / want + 31) / 32 * 32);
        n_parts = static_cast<uint32_t>((last_len + part_keys - 1) / part_keys);
    } else {
        // positions per chunk (8 S): one 8-key chunk per wavefront while the context is short (a single
        // memory round trip, many wavefronts), longer chunks once there is plenty of work.  Measured on
        // the 32/8/128 shape over rotating caches; with a kv head's query heads split over two
        // wavefronts (attn_launch_partials) 32-key chunks are best from 1024 keys up to where the split
        // ends: 64-key chunks take one wavefront per SIMD (registers) and lose 2-3 us from 8k to 16k keys.
        // heads per wavefront: attn_launch_partials has the reasons
        if (G == 8 || (G == 4 && last_len < (kv_f16 ? 32768u : 16384u))) Gw = G / 2;
        else if (G == 6) Gw = 2;
        else if (G == 3 || G == 5 || G == 7) Gw = 1;
        const bool split_heads = Gw != G;
        if (split_heads) S = last_len >= ATTN_FUSED_NEW_KV_MAX_KEYS ? 4 : 1;
        else S = last_len >= 8192 ? 8 : (last_len >= 2048 ? 4 : (last_len >= ATTN_FUSED_NEW_KV_MAX_KEYS ? 2 : 1));
        if (Gw == 8 && S == 8) S = 4;   // eight heads x 64 positions per chunk does not fit the register file
        uint32_t n_chunks = static_cast<uint32_t>((last_len + 8 * S - 1) / (8 * S));
        // parts (wavefronts) per (query, kv head): enough to fill the chip ~4 waves per CU deep
        // (more parts make the partial kernel shorter but the merge longer: measured best from 2k
        // to 128k keys with an f32 cache), but at least one chunk each and at most ATTN_MAX_PARTS
        const uint32_t waves_per_cu = kv_f16 ? 8 : 4;   // a half cache is nearer VALU-bound: more wavefronts help
        uint32_t want_parts = n_splits ? n_splits : std::max(1u, ctx->n_cu * waves_per_cu / (n_kv_heads * n_queries));
        want_parts = std::min<uint32_t>(want_parts, ATTN_MAX_PARTS);
        chunks_per_part = std::max(1u, (n_chunks + want_parts - 1) / want_parts);
        if (!n_splits) {
            // Between the lengths where that divides evenly the chip runs a ragged last round.  A
            // wavefront's time goes with its chunks, the launch's with the rounds of workgroups a CU
            // runs (one workgroup per CU and round with an f32 cache, which is bound by bytes; two with
            // an f16 cache or eight heads per kv head): from the nominal count down to a quarter of it, take the parts that
            // minimise chunks x rounds.  Of equals an f32 cache takes the one with more parts, an f16
            // cache the one with fewer -- either way the one nearer two workgroups per CU.
            // 9216 keys, f32: 31.2 -> 21.9 us together with the kernel's launch-index mapping, 13824:
            // 37.2 -> 27.9; f16: 8192 keys 16.3 -> 13.9.  Within 4 % of the best (chunk, parts) pair
            // of a sweep at every length from 1k to 16k keys (f32) and of a parts sweep (f16).
            const uint32_t subs = G / Gw;
            uint64_t best = ~0ull;
            const uint32_t first = chunks_per_part;
            for (uint32_t cpp = first; cpp <= n_chunks; ++cpp) {
                const uint64_t parts = (n_chunks + cpp - 1) / cpp;
                if (cpp > first && parts * 4 < want_parts) break;
                const uint64_t groups = (parts + 3) / 4 * n_kv_heads * subs * n_queries;   // workgroups
                // workgroups a CU takes per round: two where the kernel is bound by its own instructions
                // (an f16 cache, eight heads per kv head), one where it is bound by bytes
                const uint64_t round = static_cast<uint64_t>(ctx->n_cu) * ((kv_f16 || G == 8) ? 2 : 1);
                const uint64_t cost = cpp * ((groups + round - 1) / round);
                if (cost < best || (kv_f16 && cost == best)) { best = cost; chunks_per_part = cpp; }
            }
        }
        n_parts = (n_chunks + chunks_per_part - 1) / chunks_per_part;
    }
    uint64_t acc_bytes = static_cast<uint64_t>(n_queries) * n_kv_heads * n_parts * G * head_dim * sizeof(float);
    uint64_t ml_bytes = static_cast<uint64_t>(n_queries) * n_kv_heads * n_parts * G * 2 * sizeof(float);
    float *acc, *ml;
    if (ws) {
        // caller-provided workspace: nothing is allocated, a request that does not fit is refused
        if (acc_bytes > ws->acc_bytes || ml_bytes > ws->ml_bytes)
            return cera_fail(ctx, CERA_HIP_ERR_SHAPE,
                             "attention: the split-K partials need " + std::to_string(acc_bytes) + " + " + std::to_string(ml_bytes) +
                                 " bytes, the fixed workspace holds " + std::to_string(ws->acc_bytes) + " + " +
                                 std::to_string(ws->ml_bytes));
        acc = ws->acc;
        ml = ws->ml;
    } else {
        if (ctx->attn_acc_bytes < acc_bytes) {
            HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
            if (ctx->attn_acc) HIP_TRY(ctx, hipFree(ctx->attn_acc));
            ctx->attn_acc = nullptr; ctx->attn_acc_bytes = 0;
            HIP_TRY(ctx, hipMalloc(reinterpret_cast<void**>(&ctx->attn_acc), acc_bytes));
            ctx->attn_acc_bytes = acc_bytes;
        }
        if (ctx->attn_ml_bytes < ml_bytes) {
            HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
            if (ctx->attn_ml) HIP_TRY(ctx, hipFree(ctx->attn_ml));
            ctx->attn_ml = nullptr; ctx->attn_ml_bytes = 0;
            HIP_TRY(ctx, hipMalloc(reinterpret_cast<void**>(&ctx->attn_ml), ml_bytes));
            ctx->attn_ml_bytes = ml_bytes;
        }
        acc = ctx->attn_acc;
        ml = ctx->attn_ml;
    }
    AttnLaunch a{q, static_cast<uint32_t>(seq_len), static_cast<uint32_t>(max_seq), scale, n_heads, n_kv_heads, n_queries,
                 n_heads * head_dim, G, S, n_parts, part_keys, chunks_per_part, Gw, batch, new_kv != nullptr, nk, acc, ml};
    const kv_half *kh = static_cast<const kv_half*>(kc), *vh = static_cast<const kv_half*>(vc);
    const float *kf = static_cast<const float*>(kc), *vf = static_cast<const float*>(vc);
    if (head_dim == 128) {
        if (kv_f16) attn_launch_partials<kv_half, 128>(ctx, a, kh, vh);
        else attn_launch_partials<float, 128>(ctx, a, kf, vf);
    } else {
        if (kv_f16) attn_launch_partials<kv_half, 64>(ctx, a, kh, vh);
        else attn_launch_partials<float, 64>(ctx, a, kf, vf);
    }
    HIP_TRY(ctx, hipGetLastError());
    dim3 mgrid(n_heads, n_queries);
    const uint32_t n_pairs = n_heads * n_queries;
#define ATTN_MERGE(QQ, HH)                                                                                              \
    do {                                                                                                                \
        if (batch)                                                                                                      \
            hipLaunchKernelGGL((attn_prefill_merge_kernel<QQ, HH>), dim3((n_pairs + 7) / 8), dim3(256), 0, ctx->stream,  \
                               acc, ml, n_parts, G, n_heads, n_pairs, out, out_scales, out_quants,                      \
                               out_bsum);                                                                               \
        else                                                                                                            \
            hipLaunchKernelGGL((attn_decode_merge_kernel<QQ, HH>), mgrid, dim3(256), 0, ctx->stream, acc,                \
                               ml, n_parts, G, n_heads, out, out_scales, out_quants, out_bsum);                         \
    } while (0)
    if (out_quants) { if (head_dim == 128) ATTN_MERGE(true, 128); else ATTN_MERGE(true, 64); }
    else            { if (head_dim == 128) ATTN_MERGE(false, 128); else ATTN_MERGE(false, 64); }
#undef ATTN_MERGE
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

cera_hip_status cera_launch_attn_decode(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc,
                                        uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                        uint64_t max_seq, float scale, uint32_t n_splits, float* out,
                                        float* out_scales, int8_t* out_quants, const AttnNewKV* new_kv, bool kv_f16) {
    return cera_launch_attn(ctx, q, kc, vc, n_heads, n_kv_heads, head_dim, seq_len, max_seq, scale, n_splits, 1, out,
                            out_scales, out_quants, nullptr, new_kv, kv_f16);
}

// ---------------------------------------------------------------------------
// kernel-level entry points
extern "C" {

cera_hip_status cera_hip_quantize_q8_0_dev(cera_hip_ctx* ctx, const float* x, uint64_t k, float* scales, int8_t* quants) {
    if (!ctx || !x || !scales || !quants) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    return cera_launch_quantize(ctx, x, k, scales, quants);
}

cera_hip_status cera_hip_quantize_q8_0(cera_hip_ctx* ctx, const float* x, uint64_t k, float* scales, int8_t* quants) {
    if (!ctx || !x || !scales || !quants) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (k == 0 || k % 32) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "quantize_q8_0: k must be a positive multiple of 32");
    void *dx, *ds, *dq;
    CERA_TRY(cera_scratch(ctx, 0, k * 4, &dx));
    CERA_TRY(cera_scratch(ctx, 1, k / 32 * 4, &ds));
    CERA_TRY(cera_scratch(ctx, 2, k, &dq));
    CERA_TRY(cera_hip_upload(ctx, dx, x, k * 4));
    CERA_TRY(cera_launch_quantize(ctx, static_cast<float*>(dx), k, static_cast<float*>(ds), static_cast<int8_t*>(dq)));
    CERA_TRY(cera_hip_download(ctx, scales, ds, k / 32 * 4));
    CERA_TRY(cera_hip_download(ctx, quants, dq, k));
    return CERA_HIP_OK;
}

cera_hip_status cera_hip_gemv_q8_dev(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq, float* y) {
    if (!ctx || !w || !xs || !xq || !y) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    return cera_launch_gemv(ctx, w, nullptr, xs, xq, y, nullptr, CERA_EPI_STORE);
}

cera_hip_status cera_hip_gemv_seq_dev(cera_hip_ctx* ctx, const cera_hip_gemv_op* ops, uint32_t n) {
    if (!ctx || (!ops && n)) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    for (uint32_t i = 0; i < n; ++i) {
        if (!ops[i].w || !ops[i].xs || !ops[i].xq || !ops[i].y) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "gemv_seq: null field in op " + std::to_string(i));
        CERA_TRY(cera_launch_gemv(ctx, ops[i].w, ops[i].w2, ops[i].xs, ops[i].xq, ops[i].y, nullptr,
                                  ops[i].w2 ? CERA_EPI_SILU_MUL : CERA_EPI_STORE));
    }
    return CERA_HIP_OK;
}

cera_hip_status cera_hip_gemv(cera_hip_ctx* ctx, const cera_hip_tensor* t, const float* x, float* y,
                              int32_t* dbg_dots, int32_t* dbg_asums) {
    if (!ctx || !x || !y) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    cera_hip_dtensor* w = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, t, &w));
    cera_hip_status st = CERA_HIP_OK;
    const uint64_t k = w->k, m = w->m;
    void *dx = nullptr, *ds = nullptr, *dq = nullptr, *dy = nullptr, *dd = nullptr;
    auto run = [&]() -> cera_hip_status {
        CERA_TRY(cera_scratch(ctx, 0, k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 3, m * 4, &dy));
        CERA_TRY(cera_hip_upload(ctx, dx, x, k * 4));
        if (w->dtype == CERA_HIP_Q5_K) {
            if (dbg_dots || dbg_asums) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "Q5_K has no integer block dots (f32 activation path)");
            CERA_TRY(cera_launch_gemv_q5k_f32(ctx, w, static_cast<float*>(dx), static_cast<float*>(dy)));
        } else {
            if (!is_int8_type(w->dtype))
                return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "no gemv kernel for ggml type " + std::to_string(w->dtype));
            CERA_TRY(cera_scratch(ctx, 1, k / 32 * 4, &ds));
            CERA_TRY(cera_scratch(ctx, 2, k, &dq));
            CERA_TRY(cera_launch_quantize(ctx, static_cast<float*>(dx), k, static_cast<float*>(ds), static_cast<int8_t*>(dq)));
            uint64_t nd = (w->dtype == CERA_HIP_Q6_K ? k / 16 : k / 32);
            const bool dbg = dbg_dots || dbg_asums;
            void* da = nullptr;
            if (dbg) {
                // the debug instance accumulates partial integer dots with atomics: start from zero
                CERA_TRY(cera_scratch(ctx, 4, m * nd * 4, &dd));
                CERA_TRY(cera_scratch(ctx, 7, nd * 4, &da));
                HIP_TRY(ctx, hipMemsetAsync(dd, 0, m * nd * 4, ctx->stream));
                HIP_TRY(ctx, hipMemsetAsync(da, 0, nd * 4, ctx->stream));
            }
            CERA_TRY(cera_launch_gemv(ctx, w, nullptr, static_cast<float*>(ds), static_cast<int8_t*>(dq),
                                      static_cast<float*>(dy), nullptr, CERA_EPI_STORE, static_cast<int32_t*>(dd),
                                      static_cast<int32_t*>(da)));
            if (dbg_dots) CERA_TRY(cera_hip_download(ctx, dbg_dots, dd, m * nd * 4));
            if (dbg_asums) CERA_TRY(cera_hip_download(ctx, dbg_asums, da, nd * 4));
        }
        CERA_TRY(cera_hip_download(ctx, y, dy, m * 4));
        return CERA_HIP_OK;
    };
    st = run();
    cera_hip_tensor_free(ctx, w);
    return st;
}

cera_hip_status cera_hip_gemv_nb(cera_hip_ctx* ctx, const cera_hip_tensor* t, const float* x, uint32_t n, float* y) {
    if (!ctx || !t || !x || !y) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || t->k == 0 || t->k % 32) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemv_nb: need n > 0 and k a multiple of 32");
    cera_hip_dtensor* w = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, t, &w));
    auto run = [&]() -> cera_hip_status {
        const uint64_t k = w->k, m = w->m;
        void *dx, *ds, *dq, *dy;
        CERA_TRY(cera_scratch(ctx, 0, n * k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, n * (k / 32) * 4, &ds));
        CERA_TRY(cera_scratch(ctx, 2, n * k, &dq));
        CERA_TRY(cera_scratch(ctx, 3, n * m * 4, &dy));
        CERA_TRY(cera_hip_upload(ctx, dx, x, n * k * 4));
        // rows are multiples of 32 long, so quantizing the n rows as one vector is row by row
        CERA_TRY(cera_launch_quantize(ctx, static_cast<float*>(dx), n * k, static_cast<float*>(ds), static_cast<int8_t*>(dq)));
        // as in a model: a matrix tall enough for the streaming multi-token kernel gets its decode copy
        if (m >= 8192) CERA_TRY(cera_tensor_prepare_stream(ctx, w));
        bool launched = false;
        CERA_TRY(cera_launch_gemv_nb(ctx, w, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<uint32_t>(k / 32),
                                     static_cast<uint32_t>(k), n, static_cast<float*>(dy), static_cast<uint32_t>(m), nullptr,
                                     &launched));
        if (!launched) return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "gemv_nb: no multi-token kernel instance for this type / shape");
        return cera_hip_download(ctx, y, dy, n * m * 4);
    };
    cera_hip_status st = run();
    cera_hip_tensor_free(ctx, w);
    return st;
}

cera_hip_status cera_hip_gemv_pair(cera_hip_ctx* ctx, const cera_hip_tensor* ta, const cera_hip_tensor* tb, const float* x,
                                   float* ya, float* yb) {
    if (!ctx || !ta || !tb || !x || !ya || !yb) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (ta->k != tb->k || ta->k == 0 || ta->k % 256) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemv_pair: the two matrices must share k, a multiple of 256");
    cera_hip_dtensor *wa = nullptr, *wb = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, ta, &wa));
    cera_hip_status st = cera_hip_tensor_upload(ctx, tb, &wb);
    if (st != CERA_HIP_OK) { cera_hip_tensor_free(ctx, wa); return st; }
    auto run = [&]() -> cera_hip_status {
        const uint64_t k = wa->k;
        void *dx, *ds, *dq, *dy;
        CERA_TRY(cera_scratch(ctx, 0, k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, k / 32 * 4, &ds));
        CERA_TRY(cera_scratch(ctx, 2, k, &dq));
        CERA_TRY(cera_scratch(ctx, 3, (wa->m + wb->m) * 4, &dy));
        CERA_TRY(cera_hip_upload(ctx, dx, x, k * 4));
        CERA_TRY(cera_launch_quantize(ctx, static_cast<float*>(dx), k, static_cast<float*>(ds), static_cast<int8_t*>(dq)));
        bool launched = false;
        float *da = static_cast<float*>(dy), *db = da + wa->m;
        CERA_TRY(cera_launch_gemv_pair(ctx, wa, wb, static_cast<float*>(ds), static_cast<int8_t*>(dq), da, db, &launched));
        if (!launched) return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "gemv_pair: no paired kernel instance for these types / shapes");
        CERA_TRY(cera_hip_download(ctx, ya, da, wa->m * 4));
        return cera_hip_download(ctx, yb, db, wb->m * 4);
    };
    st = run();
    cera_hip_tensor_free(ctx, wa);
    cera_hip_tensor_free(ctx, wb);
    return st;
}

cera_hip_status cera_hip_attn_decode_dev(cera_hip_ctx* ctx, const float* q, const float* k, const float* v,
                                         uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                         uint64_t max_seq, float scale, uint32_t n_splits, float* out) {
    if (!ctx || !q || !k || !v || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    return cera_launch_attn_decode(ctx, q, k, v, n_heads, n_kv_heads, head_dim, seq_len, max_seq, scale, n_splits, out, nullptr, nullptr);
}

// Shared body of the host-pointer attention entries: n_queries consecutive queries whose first
// sees start_pos + 1 keys; K/V arrive time-major [pos][kv_dim] f32 (the reference layout) and
// are laid out head-major on the device, narrowed to half first when kv_f16.
static cera_hip_status attn_host(cera_hip_ctx* ctx, const float* q, const float* k, const float* v, uint32_t n_heads,
                                 uint32_t n_kv_heads, uint32_t head_dim, uint64_t start_pos, uint32_t n_queries,
                                 float scale, uint32_t n_splits, float* out, bool kv_f16) {
    const uint64_t seq_len = start_pos + n_queries;
    const uint64_t kv_dim = static_cast<uint64_t>(n_kv_heads) * head_dim, q_dim = static_cast<uint64_t>(n_heads) * head_dim;
    const uint64_t esz = kv_f16 ? sizeof(kv_half) : sizeof(float);
    const uint64_t kv_bytes = seq_len * kv_dim * esz, q_bytes = n_queries * q_dim * 4;
    std::vector<char> hk(kv_bytes), hv(kv_bytes);
    for (uint64_t t = 0; t < seq_len; ++t)
        for (uint32_t h = 0; h < n_kv_heads; ++h) {
            const uint64_t dst = (h * seq_len + t) * head_dim, src = t * kv_dim + h * head_dim;
            if (kv_f16) {
                for (uint32_t d = 0; d < head_dim; ++d) {
                    reinterpret_cast<kv_half*>(hk.data())[dst + d] = static_cast<kv_half>(k[src + d]);
                    reinterpret_cast<kv_half*>(hv.data())[dst + d] = static_cast<kv_half>(v[src + d]);
                }
            } else {
                std::memcpy(hk.data() + dst * 4, k + src, head_dim * 4);
                std::memcpy(hv.data() + dst * 4, v + src, head_dim * 4);
            }
        }
    void *dq, *dk, *dv, *dout;
    CERA_TRY(cera_scratch(ctx, 0, q_bytes, &dq));
    CERA_TRY(cera_scratch(ctx, 5, kv_bytes, &dk));
    CERA_TRY(cera_scratch(ctx, 6, kv_bytes, &dv));
    CERA_TRY(cera_scratch(ctx, 3, q_bytes, &dout));
    CERA_TRY(cera_hip_upload(ctx, dq, q, q_bytes));
    CERA_TRY(cera_hip_upload(ctx, dk, hk.data(), kv_bytes));
    CERA_TRY(cera_hip_upload(ctx, dv, hv.data(), kv_bytes));
    CERA_TRY(cera_launch_attn(ctx, static_cast<float*>(dq), dk, dv, n_heads, n_kv_heads, head_dim, start_pos + 1, seq_len,
                              scale, n_splits, n_queries, static_cast<float*>(dout), nullptr, nullptr, nullptr, nullptr,
                              kv_f16));
    return cera_hip_download(ctx, out, dout, q_bytes);
}

cera_hip_status cera_hip_attn_decode(cera_hip_ctx* ctx, const float* q, const float* k, const float* v,
                                     uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                     float scale, uint32_t n_splits, float* out) {
    if (!ctx || !q || !k || !v || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (seq_len == 0 || n_kv_heads == 0 || head_dim == 0) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attn_decode: empty input");
    return attn_host(ctx, q, k, v, n_heads, n_kv_heads, head_dim, seq_len - 1, 1, scale, n_splits, out, false);
}

cera_hip_status cera_hip_attn_prefill(cera_hip_ctx* ctx, const float* q, const float* k, const float* v,
                                      uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t start_pos,
                                      uint32_t n_queries, float scale, float* out) {
    if (!ctx || !q || !k || !v || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n_queries == 0 || n_kv_heads == 0 || head_dim == 0) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attn_prefill: empty input");
    return attn_host(ctx, q, k, v, n_heads, n_kv_heads, head_dim, start_pos, n_queries, scale, 0, out, false);
}

cera_hip_status cera_hip_attn_f16kv(cera_hip_ctx* ctx, const float* q, const float* k, const float* v, uint32_t n_heads,
                                    uint32_t n_kv_heads, uint32_t head_dim, uint64_t start_pos, uint32_t n_queries,
                                    float scale, uint32_t n_splits, float* out) {
    if (!ctx || !q || !k || !v || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n_queries == 0 || n_kv_heads == 0 || head_dim == 0) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attn_f16kv: empty input");
    return attn_host(ctx, q, k, v, n_heads, n_kv_heads, head_dim, start_pos, n_queries, scale, n_splits, out, true);
}

// cera_hip_attn_decode_dev without any allocation: the partials go to this device's copy of the
// static array above, through the pointer resolved at context creation.  Nothing in it has to
// start at zero (every part writes its (m, l, o) before the merge reads them), so nothing is
// cleared; calls that overlap on one GPU would share the array and race.
cera_hip_status cera_hip_attn_decode_dev_noalloc(cera_hip_ctx* ctx, const float* q, const float* k, const float* v,
                                                 uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                                 uint64_t max_seq, float scale, uint32_t n_splits, float* out) {
    if (!ctx || !q || !k || !v || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (!ctx->static_scratch) return cera_fail(ctx, CERA_HIP_ERR_DEVICE, "attn_decode_dev_noalloc: the static workspace was not resolved");
    unsigned char* base = static_cast<unsigned char*>(ctx->static_scratch);
    const AttnWorkspace ws{reinterpret_cast<float*>(base + NOALLOC_ML_BYTES), reinterpret_cast<float*>(base),
                           CERA_HIP_NOALLOC_WORKSPACE_BYTES - NOALLOC_ML_BYTES, NOALLOC_ML_BYTES};
    return cera_launch_attn(ctx, q, k, v, n_heads, n_kv_heads, head_dim, seq_len, max_seq, scale, n_splits, 1, out, nullptr,
                            nullptr, nullptr, nullptr, false, &ws);
}

cera_hip_status cera_hip_attn_decode_f16_dev(cera_hip_ctx* ctx, const float* q, const void* k16, const void* v16,
                                             uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                             uint64_t max_seq, float scale, uint32_t n_splits, float* out) {
    if (!ctx || !q || !k16 || !v16 || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    return cera_launch_attn_decode(ctx, q, k16, v16, n_heads, n_kv_heads, head_dim, seq_len, max_seq, scale, n_splits, out,
                                   nullptr, nullptr, nullptr, true);
}

cera_hip_status cera_hip_rmsnorm(cera_hip_ctx* ctx, const float* x, const float* weight, uint64_t n, float eps, float* y) {
    if (!ctx || !x || !weight || !y) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || n % 4 || n > 0xFFFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "rmsnorm: n must be a positive multiple of 4");
    void *dx, *dw, *dy;
    CERA_TRY(cera_scratch(ctx, 0, n * 4, &dx));
    CERA_TRY(cera_scratch(ctx, 1, n * 4, &dw));
    CERA_TRY(cera_scratch(ctx, 3, n * 4, &dy));
    CERA_TRY(cera_hip_upload(ctx, dx, x, n * 4));
    CERA_TRY(cera_hip_upload(ctx, dw, weight, n * 4));
    hipLaunchKernelGGL((rmsnorm_kernel<false>), dim3(1), dim3(256), 0, ctx->stream, static_cast<float*>(dx),
                       static_cast<float*>(dw), static_cast<uint32_t>(n), eps, static_cast<float*>(dy), nullptr, nullptr, nullptr);
    HIP_TRY(ctx, hipGetLastError());
    return cera_hip_download(ctx, y, dy, n * 4);
}

cera_hip_status cera_hip_silu_mul(cera_hip_ctx* ctx, const float* gate, const float* up, uint64_t n, float* out) {
    if (!ctx || !gate || !up || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || n % 4) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "silu_mul: n must be a positive multiple of 4");
    void *dg, *du, *dy;
    CERA_TRY(cera_scratch(ctx, 0, n * 4, &dg));
    CERA_TRY(cera_scratch(ctx, 1, n * 4, &du));
    CERA_TRY(cera_scratch(ctx, 3, n * 4, &dy));
    CERA_TRY(cera_hip_upload(ctx, dg, gate, n * 4));
    CERA_TRY(cera_hip_upload(ctx, du, up, n * 4));
    hipLaunchKernelGGL((silu_mul_kernel<false>), dim3(static_cast<uint32_t>((n / 4 + 255) / 256)), dim3(256), 0,
                       ctx->stream, static_cast<float*>(dg), static_cast<float*>(du), n, static_cast<float*>(dy),
                       nullptr, nullptr, nullptr);
    HIP_TRY(ctx, hipGetLastError());
    return cera_hip_download(ctx, out, dy, n * 4);
}

cera_hip_status cera_hip_argmax(cera_hip_ctx* ctx, const float* logits, uint64_t n, uint32_t* index) {
    if (!ctx || !index || (!logits && n)) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n > 0xFFFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "argmax: n exceeds 2^32");
    if (n == 0) { *index = 0; return CERA_HIP_OK; }
    void *dx, *di;
    CERA_TRY(cera_scratch(ctx, 0, n * 4, &dx));
    CERA_TRY(cera_scratch(ctx, 1, 4, &di));
    CERA_TRY(cera_hip_upload(ctx, dx, logits, n * 4));
    CERA_TRY(cera_launch_argmax(ctx, static_cast<float*>(dx), static_cast<uint32_t>(n), static_cast<uint32_t*>(di), nullptr));
    return cera_hip_download(ctx, index, di, 4);
}

cera_hip_status cera_hip_dequantize_row(cera_hip_ctx* ctx, const cera_hip_tensor* t, uint64_t row, float* out) {
    if (!ctx || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    uint64_t rb;
    CERA_TRY(check_tensor(ctx, t, &rb));
    if (row >= t->m) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "dequantize_row: row index out of range");
    void *dw, *dy, *dt;
    CERA_TRY(cera_scratch(ctx, 0, rb, &dw));
    CERA_TRY(cera_scratch(ctx, 3, t->k * 4, &dy));
    CERA_TRY(cera_scratch(ctx, 1, 4, &dt));
    CERA_TRY(cera_hip_upload(ctx, dw, static_cast<const uint8_t*>(t->data) + row * rb, rb));
    uint32_t zero = 0;
    CERA_TRY(cera_hip_upload(ctx, dt, &zero, 4));
    hipLaunchKernelGGL(embed_row_kernel, dim3(static_cast<uint32_t>((t->k + 255) / 256)), dim3(256), 0, ctx->stream,
                       t->ggml_type, static_cast<uint8_t*>(dw), rb, static_cast<uint32_t*>(dt),
                       static_cast<uint32_t>(t->k), 1.0f, static_cast<float*>(dy));
    HIP_TRY(ctx, hipGetLastError());
    return cera_hip_download(ctx, out, dy, t->k * 4);
}

}  // extern "C"
