// Public API of the llm_hip engine: the subset of PPLNN's public headers that the dynamic-batching attention path and
// its harness use, with the same class names, method names, argument meaning and error codes.
//   Engine            include/ppl/nn/engines/engine.h:30-38
//   EngineFactory     include/ppl/nn/engines/llm_cuda/engine_factory.h:36-40   (namespace llm::hip here)
//   EngineOptions     include/ppl/nn/engines/llm_cuda/engine_options.h:29-44
//   ENGINE_CONF_*     include/ppl/nn/engines/llm_cuda/options.h:33-153 (same numeric values)
//   Runtime           include/ppl/nn/runtime/runtime.h
//   Tensor            include/ppl/nn/runtime/tensor.h:28-96
//   DeviceContext     include/ppl/nn/common/device_context.h:26-44
//   RuntimeBuilder    include/ppl/nn/models/onnx/runtime_builder.h:27-76
#ifndef PPLNN_LLM_HIP_API_H_
#define PPLNN_LLM_HIP_API_H_

#include <stdarg.h>
#include <stdint.h>

#include <string>
#include <vector>

namespace ppl { namespace common {

typedef uint32_t RetCode;
enum {
    RC_SUCCESS = 0,
    RC_OTHER_ERROR,
    RC_UNSUPPORTED,
    RC_OUT_OF_MEMORY,
    RC_INVALID_VALUE,
    RC_EXISTS,
    RC_NOT_FOUND,
    RC_PERMISSION_DENIED,
    RC_HOST_MEMORY_ERROR,
    RC_DEVICE_MEMORY_ERROR,
    RC_DEVICE_RUNTIME_ERROR,
    RC_OUT_OF_RANGE,
    RC_INTERNAL_ERROR,
};
const char* GetRetCodeStr(RetCode);

typedef uint32_t datatype_t;
enum {
    DATATYPE_UNKNOWN = 0,
    DATATYPE_UINT8,
    DATATYPE_UINT16,
    DATATYPE_UINT32,
    DATATYPE_UINT64,
    DATATYPE_FLOAT16,
    DATATYPE_FLOAT32,
    DATATYPE_FLOAT64,
    DATATYPE_BFLOAT16,
    DATATYPE_INT4B,
    DATATYPE_INT8,
    DATATYPE_INT16,
    DATATYPE_INT32,
    DATATYPE_INT64,
    DATATYPE_BOOL,
};
uint32_t GetSizeOfDataType(datatype_t);
const char* GetDataTypeStr(datatype_t);

typedef uint32_t dataformat_t;
enum { DATAFORMAT_UNKNOWN = 0, DATAFORMAT_NDARRAY };

// dims + element type of an NDARRAY tensor; no padding on this path
class TensorShape final {
public:
    datatype_t GetDataType() const { return type_; }
    void SetDataType(datatype_t t) { type_ = t; }
    dataformat_t GetDataFormat() const { return DATAFORMAT_NDARRAY; }
    uint32_t GetDimCount() const { return (uint32_t)dims_.size(); }
    uint32_t GetRealDimCount() const { return scalar_ ? 0 : (uint32_t)dims_.size(); }
    int64_t GetDim(uint32_t i) const { return dims_[i]; }
    const int64_t* GetDims() const { return dims_.data(); }
    void Reshape(const int64_t* dims, uint32_t n) {
        dims_.assign(dims, dims + n);
        scalar_ = false;
    }
    void Reshape(const std::vector<int64_t>& dims) { Reshape(dims.data(), (uint32_t)dims.size()); }
    void ReshapeAsScalar() {
        dims_.assign(1, 1);
        scalar_ = true;
    }
    bool IsScalar() const { return scalar_; }
    uint64_t CalcElementsExcludingPadding() const {
        uint64_t n = 1;
        for (auto d : dims_) n *= (d < 0 ? 0 : (uint64_t)d);
        return dims_.empty() ? 0 : n;
    }
    uint64_t CalcElementsIncludingPadding() const { return CalcElementsExcludingPadding(); }
    uint64_t CalcBytesIncludingPadding() const { return CalcElementsExcludingPadding() * GetSizeOfDataType(type_); }
    uint64_t CalcBytesExcludingPadding() const { return CalcBytesIncludingPadding(); }

private:
    std::vector<int64_t> dims_;
    datatype_t type_ = DATATYPE_UNKNOWN;
    bool scalar_ = false;
};

}} // namespace ppl::common

namespace ppl { namespace nn {

using ppl::common::TensorShape;

class DeviceContext {
public:
    struct Type final {
        char str[8];
    };
    virtual ~DeviceContext() {}
    virtual const Type& GetType() const = 0;
    virtual ppl::common::RetCode Synchronize() = 0;
    virtual ppl::common::RetCode Configure(uint32_t, ...) = 0;
};

class Tensor {
public:
    virtual ~Tensor() {}
    virtual const char* GetName() const = 0;
    virtual TensorShape* GetShape() const = 0;
    virtual ppl::common::RetCode CopyToHost(void* dst) const = 0;
    virtual ppl::common::RetCode CopyToHostAsync(void* dst) const = 0;
    virtual ppl::common::RetCode CopyFromHost(const void* src) = 0;
    virtual ppl::common::RetCode CopyFromHostAsync(const void* src) = 0;
    virtual ppl::common::RetCode ConvertToHost(void* dst, const TensorShape& dst_desc) const = 0;
    virtual ppl::common::RetCode ConvertFromHost(const void* src, const TensorShape& src_desc) = 0;
    virtual DeviceContext* GetDeviceContext() const = 0;
    virtual void SetDeviceContext(DeviceContext* ctx) = 0;
    virtual void FreeBuffer() = 0;
    virtual void SetBufferPtr(void* buf) = 0;
    virtual void* GetBufferPtr() const = 0;
};

class Engine {
public:
    virtual ~Engine() {}
    virtual const char* GetName() const = 0;
    virtual ppl::common::RetCode Configure(uint32_t, ...) = 0;
};

struct ProfilingStatistics final {
    struct KernelProfilingInfo final {
        std::string kernel_name;
        std::string kernel_type;
        uint64_t exec_microseconds = 0;
        uint32_t exec_count = 0;
    };
    std::vector<KernelProfilingInfo> prof_info;
};

/** runtime options, values as in include/ppl/nn/runtime/options.h:29-47 */
enum {
    RUNTIME_CONF_SET_KERNEL_PROFILING_FLAG = 0,
    RUNTIME_CONF_INFER_SHAPES,
    RUNTIME_CONF_SET_SCHEDULER,
    RUNTIME_CONF_MAX,
};

class Runtime {
public:
    virtual ~Runtime() {}
    virtual ppl::common::RetCode Configure(uint32_t option, ...) = 0;
    virtual uint32_t GetInputCount() const = 0;
    virtual Tensor* GetInputTensor(uint32_t idx) const = 0;
    virtual ppl::common::RetCode Run() = 0;
    virtual ppl::common::RetCode RunAsync() = 0;
    virtual ppl::common::RetCode Synchronize() = 0;
    virtual uint32_t GetOutputCount() const = 0;
    virtual Tensor* GetOutputTensor(uint32_t idx) const = 0;
    virtual uint32_t GetDeviceContextCount() const = 0;
    virtual DeviceContext* GetDeviceContext(uint32_t idx) const = 0;
    virtual ppl::common::RetCode GetProfilingStatistics(ProfilingStatistics* stat) const = 0;
    virtual Tensor* GetTensor(const char* name) const = 0;
};

namespace onnx {

class RuntimeBuilder {
public:
    struct Resources final {
        Engine** engines = nullptr; // engines are managed by the caller
        uint32_t engine_num = 0;
    };
    virtual ~RuntimeBuilder() {}
    virtual ppl::common::RetCode LoadModel(const char* model_file) = 0;
    virtual ppl::common::RetCode LoadModel(const char* model_buf, uint64_t buf_len, const char* model_file_dir = nullptr) = 0;
    virtual ppl::common::RetCode SetResources(const Resources&) = 0;
    virtual ppl::common::RetCode Preprocess() = 0;
    virtual Runtime* CreateRuntime() const = 0; // thread-safe
};

class RuntimeBuilderFactory final {
public:
    static RuntimeBuilder* Create();
};

} // namespace onnx

namespace llm { namespace hip {

/** engine configuration options; numeric values of include/ppl/nn/engines/llm_cuda/options.h:33-153 */
enum {
    ENGINE_CONF_SET_TP_NCCL_COMM = 0, // accepted for source compatibility; this engine runs on one GPU -> RC_UNSUPPORTED
    ENGINE_CONF_GRAPH_FUSION = 1,
    ENGINE_CONF_TENSOR_DEBUG = 2,
    ENGINE_CONF_DEBUG_DATA_DIR = 3,
    ENGINE_CONF_MAX,
    ENGINE_CONF_INTERNAL_BEGIN = 1000,
    ENGINE_CONF_DECODING_SHM_MHA = 1000,
    ENGINE_CONF_DECODING_INF_MHA = 1001,
    ENGINE_CONF_DECODING_INF_GQA = 1002,
    ENGINE_CONF_DECODING_ATTN_SPLIT_K = 1003,
    ENGINE_CONF_DECODING_ATTN_TPB = 1004,
    ENGINE_CONF_CACHE_PREFILL = 1005,
    /** uint32_t, llm_hip only: which channels RotaryPositionEmbedding rotates together. 0 (default) = consecutive
        channels (2i, 2i+1); 1 = channel i with channel i + rotary_dim/2 ("rotate_half"). The op has no attribute for
        it and the reference's kernel is not in its tree, so the integrator states what the checkpoint was exported for */
    ENGINE_CONF_ROPE_PAIR_LAYOUT = 1006,
    /** uint32_t, llm_hip only, debugging: before MultiHeadCacheAttention trusts its tables, run the kernel library's
        table check (pplhip_check_tables) against the cache tensor's token extent, wait for it, and fail the op with
        RC_INVALID_VALUE (naming the rule and the sequence) instead of launching attention on a bad table */
    ENGINE_CONF_DEBUG_CHECK_TABLES = 1007,
    /** uint32_t, llm_hip only, debugging: wait for the stream after every op and report the op a device error belongs
        to; what the reference's debug builds do unconditionally (src/ppl/nn/engines/llm_cuda/kernel.cc:169-177) */
    ENGINE_CONF_DEBUG_SYNC_AFTER_OP = 1008,
    ENGINE_CONF_INTERNAL_MAX,
};

/** memory management policies (include/ppl/nn/engines/llm_cuda/options.h: MM_PLAIN, MM_COMPACT, MM_BEST_FIT) */
enum { MM_PLAIN, MM_COMPACT, MM_BEST_FIT };

/** device configuration options */
enum { DEV_CONF_GET_STREAM = 0, DEV_CONF_GET_DEVICE_ID, DEV_CONF_MAX };

struct EngineOptions final {
    uint32_t device_id = 0;
    uint32_t mm_policy = MM_COMPACT;
    void* runtime_stream = nullptr; // hipStream_t shared by every Runtime of this engine; nullptr = one stream per Runtime
    DeviceContext* runtime_device = nullptr;
};

struct DeviceOptions final {
    int device_id = 0;
    uint32_t mm_policy = MM_COMPACT;
    void* stream = nullptr;
};
struct HostDeviceOptions final {};

class EngineFactory final {
public:
    static Engine* Create(const EngineOptions& options);
    static DeviceContext* CreateDeviceContext(const DeviceOptions&);
    static DeviceContext* CreateHostDeviceContext(const HostDeviceOptions&);
};

}} // namespace llm::hip

// The x86 engine that runs the fp32 ONNX attention subgraph (MatMul / Mul / Add / Softmax / Transpose) on the host
// cores: the CPU baseline behind the same boundary.
//   EngineOptions / ENGINE_CONF_* / MM_*   include/ppl/nn/engines/x86/{engine_options.h:26-30, options.h:26-63}
//   EngineFactory                          include/ppl/nn/engines/x86/engine_factory.h
//   SetGlobalOmpNumThreads                 used by tools/pplnn.cc:377-380 for --num-threads
namespace x86 {

enum { ENGINE_CONF_GRAPH_FUSION = 0, ENGINE_CONF_TENSOR_DEBUG = 1, ENGINE_CONF_DEBUG_DATA_DIR = 2, ENGINE_CONF_MAX };
enum { MM_COMPACT = 0, MM_MRU = 1, MM_PLAIN = 2 };

struct EngineOptions final {
    uint32_t mm_policy = MM_COMPACT;
    bool disable_avx512 = false; // accepted; the kernels pick their instruction set at load time
    bool disable_avx_fma3 = false;
};

class EngineFactory final {
public:
    static Engine* Create(const EngineOptions&);
};

void SetGlobalOmpNumThreads(int num_threads);
int GetGlobalOmpNumThreads();

} // namespace x86

}} // namespace ppl::nn

#endif
