// The llm_hip engine: device + arena, engine / engine context, op registration and the two dynamic-batching op kernels.
// It restates, for one GPU and the attention path only,
//   engine          src/ppl/nn/engines/llm_cuda/engine.{h,cc} (Configure table :221-251, Supports :85-88, ProcessGraph :63-79)
//   engine context  src/ppl/nn/engines/llm_cuda/engine_context.cc:30-79
//   device          src/ppl/nn/engines/llm_cuda/llm_cuda_device.cc:143-221 (copies on the engine stream), buffered_device.cc:25-56
//   op base         src/ppl/nn/engines/llm_cuda/opt_kernel.h:41-139, register_ops.cc:76-85,201-206
//   kernel base     src/ppl/nn/engines/llm_cuda/kernel.cc:128-210 (event timing, error check after DoExecute)
//   MHCA op/kernel  src/ppl/nn/engines/llm_cuda/{ops,kernels}/opmx/dynamic_batching/multi_head_cache_attention_*.cc
//   KVCache op/kernel  .../key_value_cache_{op,kernel}.cc (a stub upstream; implemented here)
// All device arithmetic goes through the C ABI of libppl_llm_kernel_hip.so.
#include <hip/hip_runtime.h>

#include <fstream>
#include <mutex>

#include "arena.h"
#include "params.h"
#include "pmx_params.h"
#include "ppl_llm_kernel_hip.h"

using namespace ppl::common;

namespace ppl { namespace nn { namespace llm { namespace hip {

struct EngineConfig final { // src/ppl/nn/engines/llm_cuda/engine_config.h:25-36
    bool enable_graph_fusion = true;
    bool enable_tensor_debug = false;
    std::string debug_data_dir = ".";
    bool enable_cache_prefill = false;
    bool enable_decoding_sharemem_mhca = true;
    bool enable_decoding_infinity_mhca = true;
    bool enable_decoding_infinity_gqca = true;
    int32_t specify_decoding_attn_split_k = 1;
    int32_t specify_decoding_attn_tpb = 0;
    // which channels RotaryPositionEmbedding rotates together (PPLHIP_ROPE_PAIRS_*): not an attribute of the op, so
    // the integrator states it per engine for the checkpoint family being served
    int32_t rope_pair_layout = PPLHIP_ROPE_PAIRS_INTERLEAVED;
    // debugging aids (off by default): the device-side table check in front of MultiHeadCacheAttention, and a wait for
    // the stream after every op (the reference's debug builds: kernel.cc:169-177)
    bool debug_check_tables = false;
    bool debug_sync_after_op = false;
};

// The strides of an attn_mask tensor in the C ABI's terms: shape [S, K] (one mask for all heads) or [H, S, K] (one per
// head), K >= kvstarts[batch] (exporters pad the last extent to a multiple of 8).
// The kernels index the mask unchecked, so what can be checked on the host is: fp16 elements, one row per packed query
// token (`tokens` of them), and at least `min_keys` columns (the longest sequence's keys; the packed key total is only
// known on the device).
static RetCode MaskStrides(const TensorImpl* mask, int num_heads, int64_t tokens, int64_t min_keys, int64_t* stride_h,
                           int64_t* stride_q) {
    const TensorShape* sh = mask->GetShape();
    const uint32_t n = sh->GetDimCount();
    if (sh->GetDataType() != DATATYPE_FLOAT16) {
        LOG(ERROR) << "attn_mask must be fp16";
        return RC_INVALID_VALUE;
    }
    if (!((n == 2) || (n == 3 && (sh->GetDim(0) == num_heads || sh->GetDim(0) == 1)))) {
        LOG(ERROR) << "attn_mask must be [tokens, keys] or [num_heads, tokens, keys]";
        return RC_INVALID_VALUE;
    }
    const int64_t rows = sh->GetDim(n - 2), cols = sh->GetDim(n - 1);
    if (rows < tokens || cols < min_keys) {
        LOG(ERROR) << "attn_mask holds " << rows << " rows x " << cols << " keys; the call has " << tokens
                   << " query tokens and sequences of up to " << min_keys << " keys";
        return RC_INVALID_VALUE;
    }
    *stride_h = (n == 3 && sh->GetDim(0) != 1) ? rows * cols : 0;
    *stride_q = cols;
    return RC_SUCCESS;
}

// ---------------------------------------------------------------- device
class LlmHipDevice final : public Device {
public:
    ~LlmHipDevice() {
        arena_.reset();
        if (own_stream_ && stream_) hipStreamDestroy(stream_);
    }
    RetCode Init(int device_id, void* stream, uint32_t mm_policy = MM_BEST_FIT) {
        device_id_ = device_id;
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess || device_id >= count) {
            LOG(ERROR) << "hip device[" << device_id << "] not found (" << count << " visible)";
            return RC_NOT_FOUND;
        }
        if (hipSetDevice(device_id) != hipSuccess) return RC_DEVICE_RUNTIME_ERROR;
        if (pplhip_init() != PPLHIP_RC_SUCCESS) { // the kernel library plans its decode split for this device
            LOG(ERROR) << "kernel library init failed: " << pplhip_last_error();
            return RC_DEVICE_RUNTIME_ERROR;
        }
        if (stream) {
            stream_ = (hipStream_t)stream;
        } else {
            if (hipStreamCreate(&stream_) != hipSuccess) return RC_DEVICE_RUNTIME_ERROR; // default priority
            own_stream_ = true;
        }
        arena_.reset(new utils::ArenaBufferManager(
            [](uint64_t bytes) -> void* {
                void* p = nullptr;
                return hipMalloc(&p, bytes) == hipSuccess ? p : nullptr;
            },
            [](void* p) { (void)hipFree(p); }, 256, 64ull << 20,
            mm_policy == MM_PLAIN     ? utils::ArenaBufferManager::kPlain
                : mm_policy == MM_COMPACT ? utils::ArenaBufferManager::kCompact
                                          : utils::ArenaBufferManager::kBestFit));
        return RC_SUCCESS;
    }
    hipStream_t GetStream() const { return stream_; }
    int GetDeviceId() const { return device_id_; }
    const Type& GetType() const override {
        static const Type t = {{'h', 'i', 'p', 0, 0, 0, 0, 0}};
        return t;
    }
    RetCode Synchronize() override {
        return hipStreamSynchronize(stream_) == hipSuccess ? RC_SUCCESS : RC_DEVICE_RUNTIME_ERROR;
    }
    RetCode Configure(uint32_t option, ...) override {
        va_list args;
        va_start(args, option);
        RetCode rc = RC_SUCCESS;
        if (option == DEV_CONF_GET_STREAM) *va_arg(args, void**) = (void*)stream_;
        else if (option == DEV_CONF_GET_DEVICE_ID) *va_arg(args, int*) = device_id_;
        else rc = RC_INVALID_VALUE;
        va_end(args);
        return rc;
    }
    RetCode Realloc(uint64_t bytes, BufferDesc* buffer) override {
        if (buffer->addr && buffer->desc >= bytes) return RC_SUCCESS;
        if (buffer->addr) arena_->Free(buffer);
        if (bytes == 0) return RC_SUCCESS;
        return arena_->Alloc(bytes, buffer);
    }
    void Free(BufferDesc* buffer) override {
        if (buffer->addr) arena_->Free(buffer);
    }
    RetCode CopyFromHostAsync(BufferDesc* dst, const void* src, uint64_t bytes) const override {
        return hipMemcpyAsync(dst->addr, src, bytes, hipMemcpyHostToDevice, stream_) == hipSuccess ? RC_SUCCESS
                                                                                                   : RC_DEVICE_MEMORY_ERROR;
    }
    RetCode CopyFromHost(BufferDesc* dst, const void* src, uint64_t bytes) const override {
        auto rc = CopyFromHostAsync(dst, src, bytes);
        if (rc != RC_SUCCESS) return rc;
        return hipStreamSynchronize(stream_) == hipSuccess ? RC_SUCCESS : RC_DEVICE_RUNTIME_ERROR;
    }
    RetCode CopyToHostAsync(void* dst, const BufferDesc& src, uint64_t bytes) const override {
        return hipMemcpyAsync(dst, src.addr, bytes, hipMemcpyDeviceToHost, stream_) == hipSuccess ? RC_SUCCESS
                                                                                                  : RC_DEVICE_MEMORY_ERROR;
    }
    RetCode CopyToHost(void* dst, const BufferDesc& src, uint64_t bytes) const override {
        auto rc = CopyToHostAsync(dst, src, bytes);
        if (rc != RC_SUCCESS) return rc;
        return hipStreamSynchronize(stream_) == hipSuccess ? RC_SUCCESS : RC_DEVICE_RUNTIME_ERROR;
    }
    RetCode Copy(BufferDesc* dst, const BufferDesc& src, uint64_t bytes) const override {
        return hipMemcpyAsync(dst->addr, src.addr, bytes, hipMemcpyDeviceToDevice, stream_) == hipSuccess
            ? RC_SUCCESS
            : RC_DEVICE_MEMORY_ERROR;
    }
    // workspace of one op call, released right after the launch is enqueued (llm_cuda_device.h:151-156)
    RetCode AllocTmpBuffer(uint64_t bytes, BufferDesc* buffer) { return Realloc(bytes, buffer); }
    void FreeTmpBuffer(BufferDesc* buffer) { Free(buffer); }
    uint64_t GetBufferedBytes() const { return arena_->GetBufferedBytes(); }

private:
    int device_id_ = 0;
    hipStream_t stream_ = nullptr;
    bool own_stream_ = false;
    std::unique_ptr<utils::ArenaBufferManager> arena_;
};

class LlmHipEngineContext final : public EngineContext {
public:
    RetCode Init(const EngineOptions& options) {
        if (options.runtime_device) {
            device_ = static_cast<Device*>(options.runtime_device); // external device, managed by the caller
            return RC_SUCCESS;
        }
        owned_.reset(new LlmHipDevice());
        auto rc = owned_->Init((int)options.device_id, options.runtime_stream, options.mm_policy);
        if (rc != RC_SUCCESS) return rc;
        device_ = owned_.get();
        return RC_SUCCESS;
    }
    const char* GetName() const override { return "llm_hip"; }
    Device* GetDevice() const override { return device_; }

private:
    std::unique_ptr<LlmHipDevice> owned_;
    Device* device_ = nullptr;
};

// ---------------------------------------------------------------- kernel + op bases
class LlmHipKernel : public KernelImpl {
public:
    LlmHipKernel(const ir::Node* node, const EngineConfig* cfg) : KernelImpl(node), engine_config_(cfg) {}
    ~LlmHipKernel() {
        if (begin_) hipEventDestroy(begin_);
        if (end_) hipEventDestroy(end_);
    }
    RetCode Execute(KernelExecContext* ctx) override final {
        hipStream_t stream = GetStream();
        if (profiling_) {
            if (!begin_) {
                hipEventCreate(&begin_);
                hipEventCreate(&end_);
            }
            hipEventRecord(begin_, stream);
        }
        const RetCode rc = DoExecute(ctx);
        if (profiling_) {
            hipEventRecord(end_, stream);
            timed_ = true;
        }
        if (rc != RC_SUCCESS) return rc;
        if (GetEngineConfig().debug_sync_after_op) { // kernel.cc:169-177 (the reference's debug builds)
            const hipError_t serr = hipStreamSynchronize(stream);
            if (serr != hipSuccess) {
                LOG(ERROR) << "hipStreamSynchronize after kernel[" << GetName() << "] failed: " << (int)serr << ", "
                           << hipGetErrorString(serr);
                return RC_DEVICE_RUNTIME_ERROR;
            }
        }
        const hipError_t err = hipGetLastError(); // kernel.cc:179-185
        if (err != hipSuccess) {
            LOG(ERROR) << "exec kernel[" << GetName() << "] of type[" << GetType().domain << ":" << GetType().name
                       << "] failed: " << hipGetErrorString(err);
            return RC_DEVICE_RUNTIME_ERROR;
        }
        if (GetEngineConfig().enable_tensor_debug) { // kernel.cc:186-192
            const RetCode drc = DumpOutputTensors(ctx, GetEngineConfig().debug_data_dir);
            if (drc != RC_SUCCESS) return drc;
        }
        return RC_SUCCESS;
    }
    uint64_t GetExecutionTime() const override {
        if (!timed_) return 0;
        hipEventSynchronize(end_);
        float ms = 0;
        hipEventElapsedTime(&ms, begin_, end_);
        return (uint64_t)(ms * 1000.f);
    }
    void SetProfilingFlag(bool on) override { profiling_ = on; }

protected:
    virtual RetCode DoExecute(KernelExecContext*) = 0;
    // One file per output, named like the reference's debug dumps (engines/llm_cuda/kernel.cc:27-88) with this
    // engine's tag: <dir>/pplnn_llm_hip_dbg_tensor-<tensor name, '/' -> '.'>-<d0_d1_...|scalar|none>-<dtype>.dat.
    // The three '-'-separated parts are what the step-replay loader splits on (tools/pplnn_llm.cc:660-700).
    static RetCode DumpOutputTensors(KernelExecContext* ctx, const std::string& dir) {
        for (uint32_t i = 0; i < ctx->GetOutputCount(); ++i) {
            auto tensor = ctx->GetOutput<TensorImpl>(i);
            if (!tensor) continue;
            const std::string file = dir + "/pplnn_llm_hip_dbg_tensor-" + DumpFileTail(tensor);
            std::vector<char> host(tensor->GetShape()->CalcBytesExcludingPadding());
            auto rc = tensor->ConvertToHost(host.data(), *tensor->GetShape());
            if (rc != RC_SUCCESS) {
                LOG(ERROR) << "convert data of tensor[" << tensor->GetName() << "] failed: " << GetRetCodeStr(rc);
                return rc;
            }
            std::ofstream ofs(file, std::ios_base::out | std::ios_base::binary | std::ios_base::trunc);
            if (!ofs.is_open()) {
                LOG(ERROR) << "open output file[" << file << "] failed";
                return RC_OTHER_ERROR;
            }
            ofs.write(host.data(), host.size());
        }
        return RC_SUCCESS;
    }
    LlmHipDevice* GetHipDevice() const { return static_cast<LlmHipDevice*>(GetEngineContext()->GetDevice()); }
    hipStream_t GetStream() const { return GetHipDevice()->GetStream(); }
    const EngineConfig& GetEngineConfig() const { return *engine_config_; }
    // reads one int64 scalar; host-resident tensors (the recommended placement) cost no synchronisation
    RetCode ReadScalar(TensorImpl* t, int64_t* v) const { return t->CopyToHost(v); }

private:
    const EngineConfig* engine_config_;
    hipEvent_t begin_ = nullptr, end_ = nullptr;
    bool profiling_ = false, timed_ = false;
};

#define REQUIRED_INPUT(var, idx)                                                                         \
    auto var = ctx->GetInput<TensorImpl>(idx);                                                           \
    if (!var) {                                                                                          \
        LOG(ERROR) << "Input \"" << #var << "\" is required."; /* macros.h:84-89 */                       \
        return RC_NOT_FOUND;                                                                             \
    }
#define OPTIONAL_INPUT(var, idx) auto var = ctx->GetInputCount() > (idx) ? ctx->GetInput<TensorImpl>(idx) : nullptr
#define REQUIRED_OUTPUT(var, idx)                               \
    auto var = ctx->GetOutput<TensorImpl>(idx);                 \
    if (!var) {                                                 \
        LOG(ERROR) << "Output \"" << #var << "\" is required."; \
        return RC_NOT_FOUND;                                    \
    }
#define REALLOC_TENSOR_BUFFER(t)                                                               \
    do {                                                                                       \
        if ((t)->GetDevice() != GetHipDevice()) (t)->SetDevice(GetHipDevice()); /* macros.h:104-112 */         \
        auto rc_ = (t)->ReallocBuffer();                                                       \
        if (rc_ != RC_SUCCESS) {                                                               \
            LOG(ERROR) << "ReallocBuffer for tensor[" << (t)->GetName() << "] failed: " << GetRetCodeStr(rc_); \
            return rc_;                                                                        \
        }                                                                                      \
    } while (0)

// out shape/type := input 0 (src/ppl/nn/engines/llm_cuda/opt_kernel.h:104-115)
static RetCode GenericInferDims(InputOutputInfo* info) {
    auto in = info->GetInput<TensorImpl>(0);
    if (!in) return RC_NOT_FOUND;
    for (uint32_t i = 0; i < info->GetOutputCount(); ++i) {
        auto out = info->GetOutput<TensorImpl>(i);
        out->GetShape()->Reshape(in->GetShape()->GetDims(), in->GetShape()->GetDimCount());
        out->GetShape()->SetDataType(in->GetShape()->GetDataType());
    }
    return RC_SUCCESS;
}

static pplhip_retcode CheckKernelRc(pplhip_retcode rc, const std::string& name) {
    if (rc != PPLHIP_RC_SUCCESS) LOG(ERROR) << "kernel[" << name << "]: " << pplhip_last_error();
    return rc;
}

// ---------------------------------------------------------------- MultiHeadCacheAttention
class DynamicBatchingMultiHeadCacheAttentionKernel final : public LlmHipKernel {
public:
    DynamicBatchingMultiHeadCacheAttentionKernel(const ir::Node* node, const EngineConfig* cfg,
                                                 const opmx::MultiHeadCacheAttentionParam* p)
        : LlmHipKernel(node, cfg), param_(p) {}
    RetCode Reshape(InputOutputInfo* info) const override { return GenericInferDims(info); }

protected:
    RetCode DoExecute(KernelExecContext* ctx) override {
        REQUIRED_INPUT(query, 0);
        REQUIRED_INPUT(current_key, 1);
        REQUIRED_INPUT(current_value, 2);
        REQUIRED_INPUT(seqstarts, 3);
        REQUIRED_INPUT(kvstarts, 4);
        REQUIRED_INPUT(cachestarts, 5);
        REQUIRED_INPUT(start_pos, 6);
        REQUIRED_INPUT(decoding_batches, 7);
        REQUIRED_INPUT(max_seqlen, 8);
        REQUIRED_INPUT(max_kvlen, 9);
        REQUIRED_INPUT(cache, 10);
        OPTIONAL_INPUT(scale, 11);
        OPTIONAL_INPUT(attn_mask, 12);
        REQUIRED_OUTPUT(attn_output, 0);

        auto rc = Reshape(ctx);
        if (rc != RC_SUCCESS) return rc;

        // same checks, same order and same codes as multi_head_cache_attention_kernel.cc:90-103
        if (param_->quant_bit != 8 && param_->quant_group != 8) {
            LOG(ERROR) << "currently only support quant_bit == quant_group == 8";
            return RC_UNSUPPORTED;
        }
        if (param_->is_alibi) {
            LOG(ERROR) << "currently only support is_alibi == false";
            return RC_UNSUPPORTED;
        }
        if (!scale || scale->GetShape()->CalcElementsExcludingPadding() == 0) {
            LOG(ERROR) << "currently only support qunatized cache but scale not found";
            return RC_UNSUPPORTED;
        }
        void* attn_mask_data = nullptr;
        if (attn_mask && attn_mask->GetShape()->CalcElementsExcludingPadding() > 0) attn_mask_data = attn_mask->GetBufferPtr();

        REALLOC_TENSOR_BUFFER(attn_output);

        int64_t decoding_batches_val = 0, max_seqlen_val = 0, max_kvlen_val = 0;
        if (ReadScalar(decoding_batches, &decoding_batches_val) != RC_SUCCESS) {
            LOG(ERROR) << "decoding_batches->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        if (ReadScalar(max_seqlen, &max_seqlen_val) != RC_SUCCESS) {
            LOG(ERROR) << "max_seqlen->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        if (ReadScalar(max_kvlen, &max_kvlen_val) != RC_SUCCESS) {
            LOG(ERROR) << "max_kvlen->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        const int64_t batch = start_pos->GetShape()->GetDim(0);

        pplhip_mhca_args a;
        memset(&a, 0, sizeof(a));
        if (param_->cache_layout == 0) { // (MaxT, L, 2, H, Dh)
            a.cache_stride_s = (int64_t)param_->num_layer * 2 * param_->num_kv_heads * param_->head_dim;
            a.cache_stride_l = 2 * (int64_t)param_->num_kv_heads * param_->head_dim;
            a.cache_stride_h = param_->head_dim;
            a.cache_stride_kv = (int64_t)param_->num_kv_heads * param_->head_dim;
        } else if (param_->cache_layout == 3) { // (L, 2, H, MaxT, Dh)
            const int64_t max_tokens = cache->GetShape()->GetDim(3);
            a.cache_stride_s = param_->head_dim;
            a.cache_stride_l = 2 * (int64_t)param_->num_kv_heads * max_tokens * param_->head_dim;
            a.cache_stride_h = max_tokens * param_->head_dim;
            a.cache_stride_kv = (int64_t)param_->num_kv_heads * max_tokens * param_->head_dim;
        } else {
            LOG(ERROR) << "currently only support cache_layout == 0 or cache_layout == 3";
            return RC_UNSUPPORTED;
        }
        if (param_->cache_mode == 1) {
            if (cachestarts->GetShape()->GetDimCount() != 2) {
                LOG(ERROR) << "cachestarts must be a 2d tensor in cache_mode 1";
                return RC_INVALID_VALUE;
            }
            a.cachestart_stride_b = cachestarts->GetShape()->GetDim(1);
        }
        a.d_query = query->GetBufferPtr();
        a.d_current_key = current_key->GetBufferPtr();
        a.d_current_value = current_value->GetBufferPtr();
        a.d_attn_mask = attn_mask_data;
        if (attn_mask_data) {
            const RetCode mrc = MaskStrides(attn_mask, param_->num_heads, query->GetShape()->GetDim(0), max_kvlen_val,
                                            &a.attn_mask_stride_h, &a.attn_mask_stride_q);
            if (mrc != RC_SUCCESS) return mrc;
        }
        a.d_seqstarts = seqstarts->GetBufferPtr<int64_t>();
        a.d_kvstarts = kvstarts->GetBufferPtr<int64_t>();
        a.d_cachestarts = cachestarts->GetBufferPtr<int64_t>();
        a.d_start_pos = start_pos->GetBufferPtr<int64_t>();
        a.d_alibi_slopes = nullptr;
        a.is_causal = param_->is_causal;
        a.batch = batch;
        a.decoding_batches = decoding_batches_val;
        a.max_seqlen = max_seqlen_val;
        a.max_kvlen = max_kvlen_val;
        a.layer_idx = param_->layer_idx;
        a.num_layer = param_->num_layer;
        a.num_heads = param_->num_heads;
        a.num_kv_heads = param_->num_kv_heads;
        a.head_dim = param_->head_dim;
        a.cache_mode = param_->cache_mode;
        a.page_size = param_->page_size;
        a.enable_cache_prefill = GetEngineConfig().enable_cache_prefill;
        a.enable_decoding_sharemem_mhca = GetEngineConfig().enable_decoding_sharemem_mhca;
        a.enable_decoding_infinity_mhca = GetEngineConfig().enable_decoding_infinity_mhca;
        a.enable_decoding_infinity_gqca = GetEngineConfig().enable_decoding_infinity_gqca;
        a.specify_decoding_attn_split_k = GetEngineConfig().specify_decoding_attn_split_k;
        a.specify_decoding_attn_tpb = GetEngineConfig().specify_decoding_attn_tpb;
        a.d_cache = cache->GetBufferPtr();
        a.d_scale = scale->GetBufferPtr();
        a.d_output = attn_output->GetBufferPtr();
        a.total_new_tokens = query->GetShape()->GetDim(0);

        pplhip_mhca_plan plan;
        auto krc = CheckKernelRc(pplhip_mhca_prepare(&a, &plan), GetName());
        if (krc != PPLHIP_RC_SUCCESS) return (RetCode)krc;

        if (GetEngineConfig().debug_check_tables) {
            // token extent of the slab: dim 0 of (MaxT, L, 2, H, Dh), dim 3 of (L, 2, H, MaxT, Dh)
            const int64_t max_slab_tokens = cache->GetShape()->GetDim(param_->cache_layout == 0 ? 0 : 3);
            const RetCode trc = CheckTables(a, max_slab_tokens);
            if (trc != RC_SUCCESS) return trc;
        }

        BufferDesc tmp;
        auto status = GetHipDevice()->AllocTmpBuffer(plan.workspace_bytes, &tmp);
        if (status != RC_SUCCESS) {
            LOG(ERROR) << "alloc tmp buffer size[" << plan.workspace_bytes << "] for kernel[" << GetName()
                       << "] failed: " << GetRetCodeStr(status);
            return status;
        }
        krc = CheckKernelRc(pplhip_mhca_forward(&a, &plan, tmp.addr, GetStream()), GetName());
        // the arena hands the block to the next op on the same stream only, so stream order keeps it valid
        GetHipDevice()->FreeTmpBuffer(&tmp);
        return (RetCode)krc;
    }

private:
    // ENGINE_CONF_DEBUG_CHECK_TABLES: the kernels trust seqstarts / kvstarts / cachestarts / start_pos, and one bad entry
    // is an out-of-range slab access. The check reads the tables only; attention is not launched when it finds
    // something.
    RetCode CheckTables(const pplhip_mhca_args& a, int64_t max_slab_tokens) {
        static const char* const kRule[] = {
            "consistent", "seqstarts (must start at 0, increase, and end at the query's token count)",
            "kvstarts (must start at 0; a sequence has at least its new tokens as keys)",
            "kvlen != start_pos + seqlen (or start_pos < 0)",
            "a decode sequence must bring exactly one new token, packed at its sequence index",
            "seqlen > max_seqlen or kvlen > max_kvlen", "a slab token outside the cache tensor's token extent",
            "the page table row is shorter than the sequence's pages"};
        BufferDesc flag_buf;
        auto status = GetHipDevice()->AllocTmpBuffer(2 * sizeof(int32_t), &flag_buf);
        if (status != RC_SUCCESS) return status;
        int32_t flag[2] = {0, -1};
        auto krc = CheckKernelRc(pplhip_check_tables(&a, max_slab_tokens, (int32_t*)flag_buf.addr, GetStream()), GetName());
        if (krc == PPLHIP_RC_SUCCESS) status = GetHipDevice()->CopyToHost(flag, flag_buf, sizeof(flag)); // waits
        GetHipDevice()->FreeTmpBuffer(&flag_buf);
        if (krc != PPLHIP_RC_SUCCESS) return (RetCode)krc;
        if (status != RC_SUCCESS) return status;
        if (flag[0] != PPLHIP_TABLES_OK) {
            LOG(ERROR) << "kernel[" << GetName() << "]: inconsistent tables at sequence " << flag[1] << ": "
                       << (flag[0] > 0 && flag[0] < 8 ? kRule[flag[0]] : "unknown rule") << " (slab of "
                       << max_slab_tokens << " tokens)";
            return RC_INVALID_VALUE;
        }
        return RC_SUCCESS;
    }

    const opmx::MultiHeadCacheAttentionParam* param_;
};

// ---------------------------------------------------------------- KeyValueCache
class DynamicBatchingKeyValueCacheKernel final : public LlmHipKernel {
public:
    DynamicBatchingKeyValueCacheKernel(const ir::Node* node, const EngineConfig* cfg, const opmx::KeyValueCacheParam* p)
        : LlmHipKernel(node, cfg), param_(p) {}
    // outputs shaped like current_key with dim0 = kvstarts[B], read back from the table
    // (src/ppl/nn/oputils/opmx/reshape_dynamic_batching_key_value_cache.cc:26-53)
    RetCode Reshape(InputOutputInfo* info) const override {
        auto current_key = info->GetInput<TensorImpl>(0);
        auto kvstarts = info->GetInput<TensorImpl>(3);
        if (!current_key || !kvstarts) return RC_NOT_FOUND;
        if (!kvstarts->GetBufferPtr()) {
            LOG(DEBUG) << "ERROR: kvstarts's data is empty.";
            return RC_NOT_FOUND;
        }
        int64_t kvlen = 0;
        const uint64_t n = kvstarts->GetShape()->GetDim(0);
        BufferDesc last((char*)kvstarts->GetBufferPtr() + (n - 1) * sizeof(int64_t));
        auto rc = kvstarts->GetDevice()->CopyToHost(&kvlen, last, sizeof(int64_t));
        if (rc != RC_SUCCESS) return rc;
        std::vector<int64_t> dims(current_key->GetShape()->GetDims(),
                                  current_key->GetShape()->GetDims() + current_key->GetShape()->GetDimCount());
        dims[0] = kvlen;
        for (uint32_t i = 0; i < 2; ++i) {
            auto out = info->GetOutput<TensorImpl>(i);
            out->GetShape()->Reshape(dims);
            out->GetShape()->SetDataType(current_key->GetShape()->GetDataType());
        }
        return RC_SUCCESS;
    }

protected:
    RetCode DoExecute(KernelExecContext* ctx) override {
        REQUIRED_INPUT(current_key, 0);
        REQUIRED_INPUT(current_value, 1);
        REQUIRED_INPUT(seqstarts, 2);
        REQUIRED_INPUT(kvstarts, 3);
        REQUIRED_INPUT(cachestarts, 4);
        REQUIRED_INPUT(start_pos, 5);
        REQUIRED_INPUT(max_seqlen, 6);
        REQUIRED_INPUT(max_kvlen, 7);
        REQUIRED_INPUT(cache, 8);
        OPTIONAL_INPUT(scale, 9);
        REQUIRED_OUTPUT(key, 0);
        REQUIRED_OUTPUT(value, 1);
        (void)max_seqlen;

        auto rc = Reshape(ctx);
        if (rc != RC_SUCCESS) return rc;
        // checks of key_value_cache_kernel.cc:73-110, same order and codes
        if (!scale) {
            LOG(ERROR) << "currently only support qunatized cache but scale not found";
            return RC_UNSUPPORTED;
        }
        if (param_->quant_bit != 8 && param_->quant_group != 8) {
            LOG(ERROR) << "currently only support quant_bit == quant_group == 8";
            return RC_UNSUPPORTED;
        }
        if (param_->cache_layout != 0) {
            LOG(ERROR) << "currently only support cache_layout == 0";
            return RC_UNSUPPORTED;
        }
        if (param_->cache_mode != 0) {
            LOG(ERROR) << "currently only support cache_mode == 0";
            return RC_UNSUPPORTED;
        }
        if (param_->num_repeat != 1) {
            LOG(ERROR) << "currently only support num_repeat == 1";
            return RC_UNSUPPORTED;
        }
        REALLOC_TENSOR_BUFFER(key);
        REALLOC_TENSOR_BUFFER(value);
        if (DATATYPE_FLOAT16 != current_key->GetShape()->GetDataType()) {
            LOG(ERROR) << "currently only support fp16";
            return RC_UNSUPPORTED;
        }
        int64_t max_kvlen_val = 0;
        if (ReadScalar(max_kvlen, &max_kvlen_val) != RC_SUCCESS) return RC_DEVICE_MEMORY_ERROR;

        const int64_t kv_heads = current_key->GetShape()->GetDim(1), head_dim = current_key->GetShape()->GetDim(2);
        pplhip_kv_cache_args k;
        memset(&k, 0, sizeof(k));
        k.write.d_current_key = current_key->GetBufferPtr();
        k.write.d_current_value = current_value->GetBufferPtr();
        k.write.d_seqstarts = seqstarts->GetBufferPtr<int64_t>();
        k.write.d_cachestarts = cachestarts->GetBufferPtr<int64_t>();
        k.write.d_start_pos = start_pos->GetBufferPtr<int64_t>();
        k.write.batch = start_pos->GetShape()->GetDim(0);
        k.write.total_new_tokens = current_key->GetShape()->GetDim(0);
        k.write.layer_idx = param_->layer_idx;
        k.write.num_layer = param_->num_layer;
        k.write.num_kv_heads = (int32_t)kv_heads;
        k.write.head_dim = (int32_t)head_dim;
        k.write.cache_stride_s = (int64_t)param_->num_layer * 2 * kv_heads * head_dim;
        k.write.cache_stride_l = 2 * kv_heads * head_dim;
        k.write.cache_stride_h = head_dim;
        k.write.cache_stride_kv = kv_heads * head_dim;
        k.write.d_cache = cache->GetBufferPtr();
        k.write.d_scale = scale->GetBufferPtr();
        k.d_kvstarts = kvstarts->GetBufferPtr<int64_t>();
        k.total_kv_tokens = key->GetShape()->GetDim(0);
        k.max_kvlen = max_kvlen_val;
        k.num_repeat = param_->num_repeat;
        k.cache_mode = param_->cache_mode;
        k.cache_layout = param_->cache_layout;
        k.d_key_out = key->GetBufferPtr();
        k.d_value_out = value->GetBufferPtr();
        return (RetCode)CheckKernelRc(pplhip_kv_cache_forward(&k, GetStream()), GetName());
    }

private:
    const opmx::KeyValueCacheParam* param_;
};

// ---------------------------------------------------------------- MultiHeadAttention (no cache)
class DynamicBatchingMultiHeadAttentionKernel final : public LlmHipKernel {
public:
    DynamicBatchingMultiHeadAttentionKernel(const ir::Node* node, const EngineConfig* cfg,
                                            const opmx::MultiHeadAttentionParam* p)
        : LlmHipKernel(node, cfg), param_(p) {}
    RetCode Reshape(InputOutputInfo* info) const override { return GenericInferDims(info); }

protected:
    // inputs, checks and argument order of multi_head_attention_kernel.cc:24-128
    RetCode DoExecute(KernelExecContext* ctx) override {
        REQUIRED_INPUT(query, 0);
        REQUIRED_INPUT(key, 1);
        REQUIRED_INPUT(value, 2);
        REQUIRED_INPUT(seqstarts, 3);
        REQUIRED_INPUT(kvstarts, 4);
        REQUIRED_INPUT(decoding_batches, 5);
        REQUIRED_INPUT(max_seqlen, 6);
        REQUIRED_INPUT(max_kvlen, 7);
        OPTIONAL_INPUT(attn_mask, 8);
        REQUIRED_OUTPUT(attn_output, 0);

        auto rc = Reshape(ctx);
        if (rc != RC_SUCCESS) return rc;
        REALLOC_TENSOR_BUFFER(attn_output);
        if (param_->is_alibi) {
            LOG(ERROR) << "currently only support is_alibi == false";
            return RC_UNSUPPORTED;
        }
        int64_t decoding_batches_val = 0, max_seqlen_val = 0, max_kvlen_val = 0;
        if (ReadScalar(decoding_batches, &decoding_batches_val) != RC_SUCCESS) {
            LOG(ERROR) << "decoding_batches->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        if (ReadScalar(max_seqlen, &max_seqlen_val) != RC_SUCCESS) {
            LOG(ERROR) << "max_seqlen->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        if (ReadScalar(max_kvlen, &max_kvlen_val) != RC_SUCCESS) {
            LOG(ERROR) << "max_kvlen->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        void* attn_mask_data = nullptr;
        if (attn_mask && attn_mask->GetShape()->CalcElementsExcludingPadding() > 0) attn_mask_data = attn_mask->GetBufferPtr();

        pplhip_mha_args a;
        memset(&a, 0, sizeof(a));
        a.d_query = query->GetBufferPtr();
        a.d_key = key->GetBufferPtr();
        a.d_value = value->GetBufferPtr();
        a.d_attn_mask = attn_mask_data;
        if (attn_mask_data) {
            // (the packed keys of all sequences are the rows of `key`: the mask must have a column for each)
            const RetCode mrc = MaskStrides(attn_mask, param_->num_heads, query->GetShape()->GetDim(0),
                                            key->GetShape()->GetDim(0), &a.attn_mask_stride_h, &a.attn_mask_stride_q);
            if (mrc != RC_SUCCESS) return mrc;
        }
        a.d_seqstarts = seqstarts->GetBufferPtr<int64_t>();
        a.d_kvstarts = kvstarts->GetBufferPtr<int64_t>();
        a.is_causal = param_->is_causal;
        a.is_alibi = param_->is_alibi;
        a.batch = (int64_t)seqstarts->GetShape()->GetDim(0) - 1;
        a.decoding_batches = decoding_batches_val;
        a.max_seqlen = max_seqlen_val;
        a.max_kvlen = max_kvlen_val;
        a.num_heads = param_->num_heads;
        a.num_kv_heads = param_->num_kv_heads;
        a.head_dim = param_->head_dim;
        a.d_output = attn_output->GetBufferPtr();
        return (RetCode)CheckKernelRc(pplhip_mha_forward(&a, GetStream()), GetName());
    }

private:
    const opmx::MultiHeadAttentionParam* param_;
};

// ---------------------------------------------------------------- RotaryPositionEmbedding
class DynamicBatchingRotaryPositionEmbeddingKernel final : public LlmHipKernel {
public:
    DynamicBatchingRotaryPositionEmbeddingKernel(const ir::Node* node, const EngineConfig* cfg,
                                                 const opmx::RotaryPositionEmbeddingParam* p)
        : LlmHipKernel(node, cfg), param_(p) {}
    // oputils/opmx/reshape_rotary_position_embedding.cc:26-35
    RetCode Reshape(InputOutputInfo* info) const override {
        for (uint32_t i = 0; i < 2; ++i) {
            auto in = info->GetInput<TensorImpl>(i);
            auto out = info->GetOutput<TensorImpl>(i);
            if (!in || !out) return RC_NOT_FOUND;
            out->GetShape()->Reshape(in->GetShape()->GetDims(), in->GetShape()->GetDimCount());
            out->GetShape()->SetDataType(in->GetShape()->GetDataType());
        }
        return RC_SUCCESS;
    }

protected:
    // rotary_position_embedding_kernel.cc:24-133
    RetCode DoExecute(KernelExecContext* ctx) override {
        REQUIRED_INPUT(query, 0);
        REQUIRED_INPUT(key, 1);
        REQUIRED_INPUT(seqstarts, 2);
        REQUIRED_INPUT(start_pos, 3);
        REQUIRED_INPUT(max_seqlen, 4);
        REQUIRED_OUTPUT(rotated_query, 0);
        REQUIRED_OUTPUT(rotated_key, 1);

        auto rc = Reshape(ctx);
        if (rc != RC_SUCCESS) return rc;
        // an input this kernel is the last consumer of gives its buffer to the output (the rotation is in place)
        void* query_data = query->GetBufferPtr();
        void* key_data = key->GetBufferPtr();
        if (ctx->IsLastConsumerOfInput(0) && query->GetBufferInfo().IsBufferOwner()) {
            rotated_query->TransferBufferFrom(query);
        } else {
            REALLOC_TENSOR_BUFFER(rotated_query);
        }
        if (ctx->IsLastConsumerOfInput(1) && key->GetBufferInfo().IsBufferOwner()) {
            rotated_key->TransferBufferFrom(key);
        } else {
            REALLOC_TENSOR_BUFFER(rotated_key);
        }
        auto query_shape = rotated_query->GetShape();
        auto key_shape = rotated_key->GetShape();
        if (DATATYPE_FLOAT16 != query_shape->GetDataType()) {
            LOG(ERROR) << "currently only support fp16";
            return RC_UNSUPPORTED;
        }
        int64_t max_seqlen_val = 0;
        if (ReadScalar(max_seqlen, &max_seqlen_val) != RC_SUCCESS) {
            LOG(ERROR) << "max_seqlen->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        // The reference maps the parameter through `!=` tests (rotary_position_embedding_kernel.cc:99-108), which
        // turns NONE into LINEAR and LINEAR / DYNAMIC into NONE; the value is taken at its name here.
        int32_t scaling_type;
        if (param_->scaling_type == param_->SCALING_TYPE_NONE) {
            scaling_type = PPLHIP_ROPE_SCALING_NONE;
        } else if (param_->scaling_type == param_->SCALING_TYPE_LINEAR) {
            scaling_type = PPLHIP_ROPE_SCALING_LINEAR;
        } else if (param_->scaling_type == param_->SCALING_TYPE_DYNAMIC) {
            scaling_type = PPLHIP_ROPE_SCALING_DYNAMIC;
        } else {
            LOG(ERROR) << "invalid scaling type: " << param_->scaling_type;
            return RC_INVALID_VALUE;
        }
        pplhip_rope_args a;
        memset(&a, 0, sizeof(a));
        a.d_query = query_data;
        a.d_key = key_data;
        a.d_start_pos = start_pos->GetBufferPtr<int64_t>();
        a.d_seqstarts = seqstarts->GetBufferPtr<int64_t>();
        a.theta = param_->theta;
        a.bypass_key = param_->bypass_key;
        a.head_dim = (int32_t)query_shape->GetDim(2);
        a.rotary_dim = param_->rotary_dim == 0 ? a.head_dim : param_->rotary_dim;
        a.batch = start_pos->GetShape()->GetDim(0);
        a.total_tokens = query_shape->GetDim(0);
        a.num_heads = (int32_t)query_shape->GetDim(1);
        a.num_key_heads = (int32_t)key_shape->GetDim(1);
        a.max_position_embeddings = param_->max_position_embeddings;
        a.max_seqlen = max_seqlen_val;
        a.scaling_type = scaling_type;
        a.scaling_factor = param_->scaling_factor;
        a.pair_layout = GetEngineConfig().rope_pair_layout;
        a.d_rotated_query = rotated_query->GetBufferPtr();
        a.d_rotated_key = rotated_key->GetBufferPtr();
        return (RetCode)CheckKernelRc(pplhip_rope_forward(&a, GetStream()), GetName());
    }

private:
    const opmx::RotaryPositionEmbeddingParam* param_;
};

// ---------------------------------------------------------------- PositionIndex
class DynamicBatchingPositionIndexKernel final : public LlmHipKernel {
public:
    DynamicBatchingPositionIndexKernel(const ir::Node* node, const EngineConfig* cfg) : LlmHipKernel(node, cfg) {}
    RetCode Reshape(InputOutputInfo* info) const override { return GenericInferDims(info); }

protected:
    // position_index_kernel.cc:24-70
    RetCode DoExecute(KernelExecContext* ctx) override {
        REQUIRED_INPUT(sequence, 0);
        REQUIRED_INPUT(seqstarts, 1);
        REQUIRED_INPUT(start_pos, 2);
        REQUIRED_INPUT(max_seqlen, 3);
        REQUIRED_OUTPUT(position_idx, 0);

        auto rc = Reshape(ctx);
        if (rc != RC_SUCCESS) return rc;
        if (ctx->IsLastConsumerOfInput(0) && sequence->GetBufferInfo().IsBufferOwner()) {
            position_idx->TransferBufferFrom(sequence);
        } else {
            REALLOC_TENSOR_BUFFER(position_idx);
        }
        if (DATATYPE_INT64 != position_idx->GetShape()->GetDataType()) {
            LOG(ERROR) << "position_idx takes the type of the token sequence, which must be int64";
            return RC_UNSUPPORTED;
        }
        int64_t max_seqlen_val = 0;
        if (ReadScalar(max_seqlen, &max_seqlen_val) != RC_SUCCESS) {
            LOG(ERROR) << "max_seqlen->CopyToHost() failed";
            return RC_DEVICE_MEMORY_ERROR;
        }
        const int64_t batch = start_pos->GetShape()->GetDim(0);
        const int64_t total = (int64_t)position_idx->GetShape()->CalcElementsExcludingPadding();
        return (RetCode)CheckKernelRc(
            pplhip_position_index(start_pos->GetBufferPtr<int64_t>(), seqstarts->GetBufferPtr<int64_t>(), batch, total,
                                  max_seqlen_val, position_idx->GetBufferPtr<int64_t>(), GetStream()),
            GetName());
    }
};

// ---------------------------------------------------------------- ops + registry
class LlmHipOptKernel : public OptKernel {
public:
    LlmHipOptKernel(const ir::Node* node) : OptKernel(node) {}
    virtual RetCode Init(const ir::Graph* graph, const EngineConfig* cfg) = 0;

protected:
    template <typename T>
    RetCode GenericLoadParam(const ir::Graph* graph, std::shared_ptr<T>* param) { // opt_kernel.h:50-61
        auto it = graph->data->attrs.find(GetNode()->GetId());
        if (it == graph->data->attrs.end()) {
            LOG(ERROR) << "cannot find attr for op[" << GetNode()->GetName() << "]";
            return RC_NOT_FOUND;
        }
        *param = std::static_pointer_cast<T>(it->second);
        return RC_SUCCESS;
    }
    const EngineConfig* cfg_ = nullptr;
};

class DynamicBatchingMultiHeadCacheAttentionOp final : public LlmHipOptKernel {
public:
    using LlmHipOptKernel::LlmHipOptKernel;
    RetCode Init(const ir::Graph* graph, const EngineConfig* cfg) override {
        cfg_ = cfg;
        return GenericLoadParam(graph, &param_);
    }
    KernelImpl* CreateKernelImpl() const override {
        return new DynamicBatchingMultiHeadCacheAttentionKernel(GetNode(), cfg_, param_.get());
    }

    RetCode SerializeData(std::string* blob) const override {
        *blob = pmx::SerializeOpParam(*param_);
        return RC_SUCCESS;
    }
    RetCode DeserializeData(const void* base, uint64_t size) override {
        param_ = std::make_shared<opmx::MultiHeadCacheAttentionParam>();
        return pmx::DeserializeOpParam(base, size, param_.get());
    }

private:
    std::shared_ptr<opmx::MultiHeadCacheAttentionParam> param_;
};

class DynamicBatchingKeyValueCacheOp final : public LlmHipOptKernel {
public:
    using LlmHipOptKernel::LlmHipOptKernel;
    RetCode Init(const ir::Graph* graph, const EngineConfig* cfg) override {
        cfg_ = cfg;
        return GenericLoadParam(graph, &param_);
    }
    KernelImpl* CreateKernelImpl() const override {
        return new DynamicBatchingKeyValueCacheKernel(GetNode(), cfg_, param_.get());
    }

    RetCode SerializeData(std::string* blob) const override {
        *blob = pmx::SerializeOpParam(*param_);
        return RC_SUCCESS;
    }
    RetCode DeserializeData(const void* base, uint64_t size) override {
        param_ = std::make_shared<opmx::KeyValueCacheParam>();
        return pmx::DeserializeOpParam(base, size, param_.get());
    }

private:
    std::shared_ptr<opmx::KeyValueCacheParam> param_;
};

class DynamicBatchingMultiHeadAttentionOp final : public LlmHipOptKernel {
public:
    using LlmHipOptKernel::LlmHipOptKernel;
    RetCode Init(const ir::Graph* graph, const EngineConfig* cfg) override {
        cfg_ = cfg;
        return GenericLoadParam(graph, &param_);
    }
    KernelImpl* CreateKernelImpl() const override {
        return new DynamicBatchingMultiHeadAttentionKernel(GetNode(), cfg_, param_.get());
    }

    RetCode SerializeData(std::string* blob) const override {
        *blob = pmx::SerializeOpParam(*param_);
        return RC_SUCCESS;
    }
    RetCode DeserializeData(const void* base, uint64_t size) override {
        param_ = std::make_shared<opmx::MultiHeadAttentionParam>();
        return pmx::DeserializeOpParam(base, size, param_.get());
    }

private:
    std::shared_ptr<opmx::MultiHeadAttentionParam> param_;
};

class DynamicBatchingRotaryPositionEmbeddingOp final : public LlmHipOptKernel {
public:
    using LlmHipOptKernel::LlmHipOptKernel;
    RetCode Init(const ir::Graph* graph, const EngineConfig* cfg) override {
        cfg_ = cfg;
        return GenericLoadParam(graph, &param_);
    }
    KernelImpl* CreateKernelImpl() const override {
        return new DynamicBatchingRotaryPositionEmbeddingKernel(GetNode(), cfg_, param_.get());
    }

    RetCode SerializeData(std::string* blob) const override {
        *blob = pmx::SerializeOpParam(*param_);
        return RC_SUCCESS;
    }
    RetCode DeserializeData(const void* base, uint64_t size) override {
        param_ = std::make_shared<opmx::RotaryPositionEmbeddingParam>();
        return pmx::DeserializeOpParam(base, size, param_.get());
    }

private:
    std::shared_ptr<opmx::RotaryPositionEmbeddingParam> param_;
};

class DynamicBatchingPositionIndexOp final : public LlmHipOptKernel { // no attributes (position_index_op.cc:29-41)
public:
    using LlmHipOptKernel::LlmHipOptKernel;
    RetCode Init(const ir::Graph*, const EngineConfig* cfg) override {
        cfg_ = cfg;
        return RC_SUCCESS;
    }
    KernelImpl* CreateKernelImpl() const override { return new DynamicBatchingPositionIndexKernel(GetNode(), cfg_); }
};

typedef LlmHipOptKernel* (*OptKernelCreator)(const ir::Node*);

utils::OpInfoManager<OptKernelCreator>& OptKernelCreatorManager() {
    static utils::OpInfoManager<OptKernelCreator> mgr;
    return mgr;
}

template <typename T>
static LlmHipOptKernel* GenericCreateOptKernel(const ir::Node* node) {
    return new T(node);
}

template <typename T>
static void RegisterOptKernelCreator(const std::string& domain, const std::string& type, uint64_t first, uint64_t last) {
    if (last < first) { // register_ops.cc:78-82
        LOG(ERROR) << "register op[" << domain << ":" << type << "] failed: last version[" << last
                   << "] < first version[" << first << "]";
        exit(-1);
    }
    OptKernelCreatorManager().Register(domain, type, utils::VersionRange{first, last}, GenericCreateOptKernel<T>);
}

static void RegisterResourcesOnce() { // default_register_resources.cc:28-34
    static std::once_flag once;
    std::call_once(once, [] {
        RegisterOptKernelCreator<DynamicBatchingKeyValueCacheOp>("opmx.dynamic_batching", "KeyValueCache", 1, 1);
        RegisterOptKernelCreator<DynamicBatchingMultiHeadCacheAttentionOp>("opmx.dynamic_batching", "MultiHeadCacheAttention", 1, 1);
        RegisterOptKernelCreator<DynamicBatchingMultiHeadAttentionOp>("opmx.dynamic_batching", "MultiHeadAttention", 1, 1);
        RegisterOptKernelCreator<DynamicBatchingPositionIndexOp>("opmx.dynamic_batching", "PositionIndex", 1, 1);
        RegisterOptKernelCreator<DynamicBatchingRotaryPositionEmbeddingOp>("opmx.dynamic_batching", "RotaryPositionEmbedding", 1, 1);
    });
}

// ---------------------------------------------------------------- engine
class LlmHipEngine final : public EngineImpl {
public:
    LlmHipEngine() : EngineImpl("llm_hip") {}
    RetCode Init(const EngineOptions& options) {
        options_ = options;
        if (options.mm_policy != MM_PLAIN && options.mm_policy != MM_COMPACT && options.mm_policy != MM_BEST_FIT) {
            LOG(ERROR) << "unknown mm_policy " << options.mm_policy;
            return RC_INVALID_VALUE;
        }
        return RC_SUCCESS;
    }
    EngineContext* CreateEngineContext() override {
        auto ctx = new LlmHipEngineContext();
        if (ctx->Init(options_) != RC_SUCCESS) {
            delete ctx;
            return nullptr;
        }
        return ctx;
    }
    bool Supports(const ir::Node* node) const override {
        auto& type = node->GetType();
        return OptKernelCreatorManager().Find(type.domain, type.name, type.version) != nullptr;
    }
    RetCode ProcessGraph(ir::Graph* graph, RuntimePartitionInfo* info) override {
        for (auto& node : graph->topo->nodes) { // OptGraph::Init (create ops) + Optimize (init ops), opt_graph.cc:31-160
            auto& type = node.GetType();
            auto creator = OptKernelCreatorManager().Find(type.domain, type.name, type.version);
            if (!creator) {
                LOG(ERROR) << "cannot find creator for node[" << node.GetName() << "] of type[" << type.domain << ":"
                           << type.name << ":" << type.version << "]";
                return RC_NOT_FOUND;
            }
            std::unique_ptr<LlmHipOptKernel> op((*creator)(&node));
            auto rc = op->Init(graph, &config_);
            if (rc != RC_SUCCESS) {
                LOG(ERROR) << "Init for kernel[" << node.GetName() << "] failed: " << GetRetCodeStr(rc);
                return rc;
            }
            info->kernels[node.GetId()] = std::move(op);
        }
        return RC_SUCCESS;
    }
    RetCode Configure(uint32_t option, ...) override { // engine.cc:236-251: internal options are remapped
        va_list args;
        va_start(args, option);
        RetCode rc = RC_SUCCESS;
        switch (option) {
            case ENGINE_CONF_SET_TP_NCCL_COMM:
                LOG(ERROR) << "this engine runs on one GPU: tensor-parallel communicators are not supported";
                rc = RC_UNSUPPORTED;
                break;
            case ENGINE_CONF_GRAPH_FUSION: config_.enable_graph_fusion = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_TENSOR_DEBUG: config_.enable_tensor_debug = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_DEBUG_DATA_DIR: config_.debug_data_dir = va_arg(args, const char*); break;
            case ENGINE_CONF_DECODING_SHM_MHA: config_.enable_decoding_sharemem_mhca = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_DECODING_INF_MHA: config_.enable_decoding_infinity_mhca = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_DECODING_INF_GQA: config_.enable_decoding_infinity_gqca = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_DECODING_ATTN_SPLIT_K: {
                const uint32_t v = va_arg(args, uint32_t);
                if (v > 2) { // engine.cc:150-170
                    LOG(ERROR) << "ENGINE_CONF_DECODING_ATTN_SPLIT_K only accept 0/1/2 but get " << v;
                    rc = RC_INVALID_VALUE;
                } else {
                    config_.specify_decoding_attn_split_k = (int32_t)v;
                }
                break;
            }
            case ENGINE_CONF_DECODING_ATTN_TPB: {
                const uint32_t v = va_arg(args, uint32_t);
                if (v != 0 && v != 256 && v != 512) {
                    LOG(ERROR) << "ENGINE_CONF_DECODING_ATTN_TPB only accept 0/256/512 but get " << v;
                    rc = RC_INVALID_VALUE;
                } else {
                    config_.specify_decoding_attn_tpb = (int32_t)v;
                }
                break;
            }
            case ENGINE_CONF_CACHE_PREFILL: config_.enable_cache_prefill = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_ROPE_PAIR_LAYOUT: {
                const uint32_t v = va_arg(args, uint32_t);
                if (v != PPLHIP_ROPE_PAIRS_INTERLEAVED && v != PPLHIP_ROPE_PAIRS_HALF_SPLIT) {
                    LOG(ERROR) << "ENGINE_CONF_ROPE_PAIR_LAYOUT only accept 0/1 but get " << v;
                    rc = RC_INVALID_VALUE;
                } else {
                    config_.rope_pair_layout = (int32_t)v;
                }
                break;
            }
            case ENGINE_CONF_DEBUG_CHECK_TABLES: config_.debug_check_tables = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_DEBUG_SYNC_AFTER_OP: config_.debug_sync_after_op = va_arg(args, uint32_t) ? true : false; break;
            default:
                LOG(ERROR) << "invalid option[" << option << "] >= [" << (uint32_t)ENGINE_CONF_INTERNAL_MAX << "]";
                rc = RC_INVALID_VALUE;
        }
        va_end(args);
        if (rc == RC_SUCCESS && !config_.enable_decoding_sharemem_mhca && !config_.enable_decoding_infinity_mhca &&
            !config_.enable_decoding_infinity_gqca)
            LOG(WARNING) << "all decoding attention algorithms are disabled; the single algorithm of this engine is used anyway";
        return rc;
    }
    const EngineConfig& GetEngineConfig() const { return config_; }

private:
    EngineOptions options_;
    EngineConfig config_;
};

Engine* EngineFactory::Create(const EngineOptions& options) {
    RegisterResourcesOnce();
    auto engine = new LlmHipEngine();
    auto rc = engine->Init(options);
    if (rc != RC_SUCCESS) {
        LOG(ERROR) << "init llm_hip engine failed: " << GetRetCodeStr(rc);
        delete engine;
        return nullptr;
    }
    return engine;
}

DeviceContext* EngineFactory::CreateDeviceContext(const DeviceOptions& options) {
    auto dev = new LlmHipDevice();
    if (dev->Init(options.device_id, options.stream, options.mm_policy) != RC_SUCCESS) {
        delete dev;
        return nullptr;
    }
    return dev;
}

namespace {
class HostDeviceHandle final : public Device { // a caller-owned handle onto the shared host device
public:
    const Type& GetType() const override { return GetSharedHostDevice()->GetType(); }
    RetCode Synchronize() override { return RC_SUCCESS; }
    RetCode Configure(uint32_t, ...) override { return RC_UNSUPPORTED; }
    RetCode Realloc(uint64_t bytes, BufferDesc* b) override { return GetSharedHostDevice()->Realloc(bytes, b); }
    void Free(BufferDesc* b) override { GetSharedHostDevice()->Free(b); }
    RetCode CopyFromHost(BufferDesc* d, const void* s, uint64_t n) const override { return GetSharedHostDevice()->CopyFromHost(d, s, n); }
    RetCode CopyFromHostAsync(BufferDesc* d, const void* s, uint64_t n) const override { return GetSharedHostDevice()->CopyFromHost(d, s, n); }
    RetCode CopyToHost(void* d, const BufferDesc& s, uint64_t n) const override { return GetSharedHostDevice()->CopyToHost(d, s, n); }
    RetCode CopyToHostAsync(void* d, const BufferDesc& s, uint64_t n) const override { return GetSharedHostDevice()->CopyToHost(d, s, n); }
    RetCode Copy(BufferDesc* d, const BufferDesc& s, uint64_t n) const override { return GetSharedHostDevice()->Copy(d, s, n); }
};
} // namespace

DeviceContext* EngineFactory::CreateHostDeviceContext(const HostDeviceOptions&) {
    return new HostDeviceHandle();
}

}}}} // namespace ppl::nn::llm::hip
