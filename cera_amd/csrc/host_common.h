// Host-side types shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "attn_types.h"
#include "cera_hip.h"

struct cera_hip_event {
    hipEvent_t ev = nullptr;
};

struct cera_hip_dtensor {
    uint32_t dtype = 0;
    uint64_t m = 0, k = 0;
    uint64_t row_bytes = 0, nbytes = 0;
    uint8_t* dev = nullptr;
    bool owns = true;  // false: a row-range view into another tensor's allocation
    // optional decode copy (cera_tensor_prepare_stream): the rows permuted for streaming reads,
    // row stride stream_row_bytes; owned by this tensor
    uint8_t* dev_stream = nullptr;
    uint64_t stream_row_bytes = 0;
};

struct cera_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::string err;
    uint32_t n_cu = 0;
    bool decode_copies = true;   // cera_hip_ctx_set_decode_copies
    // serialises every call that uses the stream's workspaces below (kernel-level entry points
    // with host buffers, and every model-level call of any model on this context)
    std::recursive_mutex op_mu;
    // grow-only device scratch for the host-pointer entry points
    void* scratch[16] = {nullptr};
    uint64_t scratch_bytes[16] = {0};
    void* static_scratch = nullptr;   // this device's copy of the library's fixed workspace (resolved at creation)
    // optional standalone code object (cera_hip_ctx_create with an hsaco_path): the quantizer and the
    // GEMV instances it exports are then launched from it with hipModuleLaunchKernel
    hipModule_t module = nullptr;
    std::unordered_map<std::string, hipFunction_t> module_fns;   // name -> function, nullptr = not exported
    // attention split-K workspace
    float* attn_acc = nullptr;
    float* attn_ml = nullptr;
    uint64_t attn_acc_bytes = 0, attn_ml_bytes = 0;
    // two pinned chunks + events: staging for device-to-host copies into pageable memory
    std::mutex pin_mu;
    void* pin[2] = {nullptr, nullptr};
    hipEvent_t pin_ev[2] = {nullptr, nullptr};
    // one pinned word the device writes directly (the greedy step's token): host view and device view
    uint32_t* word_host = nullptr;
    uint32_t* word_dev = nullptr;
};

void cera_set_global_error(const std::string& s);
cera_hip_status cera_fail(cera_hip_ctx* ctx, cera_hip_status st, const std::string& msg);

#define HIP_TRY(ctx, call)                                                                     \
    do {                                                                                       \
        hipError_t e_ = (call);                                                                \
        if (e_ != hipSuccess)                                                                  \
            return cera_fail((ctx), e_ == hipErrorOutOfMemory ? CERA_HIP_ERR_OOM : CERA_HIP_ERR_DEVICE, \
                             std::string(#call) + ": " + hipGetErrorString(e_));               \
    } while (0)

#define CERA_TRY(expr)                          \
    do {                                        \
        cera_hip_status s_ = (expr);            \
        if (s_ != CERA_HIP_OK) return s_;       \
    } while (0)

// element / byte geometry of a GGML type; false when there is no kernel for it
bool cera_type_geometry(uint32_t t, uint32_t* block_elems, uint32_t* block_bytes);
cera_hip_status cera_scratch(cera_hip_ctx* ctx, int slot, uint64_t nbytes, void** out);
// kernel `name` of the context's loaded code object, nullptr when there is no module or no such kernel
hipFunction_t cera_module_fn(cera_hip_ctx* ctx, const std::string& name);
// launch a one-struct-argument kernel of the loaded code object
cera_hip_status cera_module_launch(cera_hip_ctx* ctx, hipFunction_t f, uint32_t grid, uint32_t block, void* args);

// ---- launchers (defined next to their kernels) --------------------------------
enum CeraEpilogue { CERA_EPI_STORE = 0, CERA_EPI_ADD = 1, CERA_EPI_SILU_MUL = 2 };

cera_hip_status cera_launch_quantize(cera_hip_ctx* ctx, const float* x, uint64_t k, float* scales, int8_t* quants,
                                     float* bsum = nullptr);
// y = W.(xs,xq) [+ resid]; w2 != null with EPI_SILU_MUL computes silu(W.x)*(W2.x)
cera_hip_status cera_launch_gemv(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const cera_hip_dtensor* w2,
                                 const float* xs, const int8_t* xq, float* y, const float* resid, int epi,
                                 int32_t* dbg_dots = nullptr, int32_t* dbg_asums = nullptr);
// y = resid + W.(xs,xq) with one wavefront per row; *launched = false when the shape has no such instance
cera_hip_status cera_launch_row_gemv_add(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                         float* y, const float* resid, bool* launched);
cera_hip_status cera_tensor_prepare_stream(cera_hip_ctx* ctx, cera_hip_dtensor* w);
// bytes a decode copy of w would take (0: none possible, or it has one); free an existing one
uint64_t cera_tensor_stream_bytes(const cera_hip_ctx* ctx, const cera_hip_dtensor* w);
void cera_tensor_drop_stream(cera_hip_dtensor* w);
cera_hip_status cera_launch_row_gemv_store(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                           float* y, bool* launched);
cera_hip_status cera_launch_row_gemv_long_add(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                              float* y, const float* resid, bool* launched);
cera_hip_status cera_launch_gemv_nb(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                    uint32_t xs_stride, uint32_t xq_stride, uint32_t n_tok, float* y, uint32_t y_stride,
                                    const float* resid, bool* launched);
cera_hip_status cera_launch_row_gemv_nb(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                    uint32_t xs_stride, uint32_t xq_stride, uint32_t n_tok, float* y, uint32_t y_stride,
                                    const float* resid, bool* launched);
cera_hip_status cera_launch_gemv_pair(cera_hip_ctx* ctx, const cera_hip_dtensor* wa, const cera_hip_dtensor* wb,
                                      const float* xs, const int8_t* xq, float* ya, float* yb, bool* launched);
// Decode projections with the neighbouring small kernels folded in (gemv_fused.hip); *launched =
// false when the shapes / types have no fused instance and the caller takes the separate launches.
//   gate|up: out_q / out_s = Q8_0(silu(gate . n) * (up . n)), n = Q8_0(rmsnorm(x, norm_w))
//   q|k|v:   ya = A . n, yb = B . n (wb nullable)
cera_hip_status cera_launch_ffn_gate_up_fused(cera_hip_ctx* ctx, const cera_hip_dtensor* gate, const cera_hip_dtensor* up,
                                              const float* x, const float* norm_w, float eps, int8_t* out_q, float* out_s,
                                              bool* launched);
cera_hip_status cera_launch_qkv_fused(cera_hip_ctx* ctx, const cera_hip_dtensor* wa, const cera_hip_dtensor* wb, const float* x,
                                      const float* norm_w, float eps, float* ya, float* yb, bool* launched);
// one query, any head_dim % 8 == 0 up to 256, any heads per kv head (reforder.hip); scores: [n_heads][max_seq] floats
cera_hip_status cera_launch_attn_generic(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc, uint32_t n_heads,
                                         uint32_t n_kv_heads, uint32_t head_dim, uint32_t seq_len, uint32_t max_seq, float scale,
                                         float* scores, float* out, bool kv_f16);
// whether the tuned attention kernels cover the shape (else cera_launch_attn takes the generic kernel per query)
static inline bool cera_attn_shape_tuned(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim) {
    return (head_dim == 64 || head_dim == 128) && n_kv_heads != 0 && n_heads % n_kv_heads == 0 && n_heads / n_kv_heads <= 8;
}
// index of the maximum of x[0, n) into *out_dev (device); uses scratch slot 8 of the context
// out_host_mapped (nullable): device view of pinned host memory that also receives the index
cera_hip_status cera_launch_argmax(cera_hip_ctx* ctx, const float* x, uint32_t n, uint32_t* out_dev, uint32_t* out_host_mapped);
// the context's pinned word (allocated at first use)
cera_hip_status cera_pinned_word(cera_hip_ctx* ctx, uint32_t** host, uint32_t** dev);
cera_hip_status cera_launch_gemv_q5k_f32(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* x, float* y);
// kc / vc: [n_kv_heads][max_seq][head_dim], f32 or IEEE half (kv_f16)
cera_hip_status cera_launch_attn_decode(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc,
                                        uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                        uint64_t max_seq, float scale, uint32_t n_splits, float* out,
                                        float* out_scales, int8_t* out_quants, const AttnNewKV* new_kv = nullptr,
                                        bool kv_f16 = false);
// where the split-K partials of an attention launch go when the caller provides the memory
struct AttnWorkspace {
    float* acc;   // [query][kv head][part][group][head_dim]
    float* ml;    // [query][kv head][part][group][2]
    uint64_t acc_bytes, ml_bytes;
};
// n_queries consecutive queries (causal): query i sees seq_len + i keys; q and the outputs are
// [n_queries][n_heads*head_dim].  ws == null: the context's own grow-on-demand workspace.
cera_hip_status cera_launch_attn(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc,
                                 uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                 uint64_t max_seq, float scale, uint32_t n_splits, uint32_t n_queries, float* out,
                                 float* out_scales, int8_t* out_quants, float* out_bsum,
                                 const AttnNewKV* new_kv = nullptr, bool kv_f16 = false,
                                 const AttnWorkspace* ws = nullptr);
// One allocation holding the rows of several same-type, same-k matrices back to back
// (`fused`), plus a non-owning view per part.  Lets the decode step run Q|K(|V) as one GEMV.
cera_hip_status cera_tensor_upload_concat(cera_hip_ctx* ctx, const cera_hip_tensor* const* parts, int n_parts,
                                          cera_hip_dtensor** fused, cera_hip_dtensor** views);
