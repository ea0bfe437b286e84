// Internal boundary types of the llm_hip host engine, shaped after the reference's plug-in boundary:
//   ir::Node / Edge / Graph / Attr        src/ppl/nn/ir/{node.h:29-45, edge.h, graph.h, attr.h:6-16}
//   OpInfoManager                         src/ppl/nn/utils/op_info_manager.h:36-115
//   Device / BufferDesc                   src/ppl/nn/common/device.h:30-137, buffer_desc.h:25-36
//   BufferInfo / TensorImpl               src/ppl/nn/common/buffer_info.cc:65-113, src/ppl/nn/runtime/tensor_impl.{h,cc}
//   InputOutputInfo / KernelExecContext   src/ppl/nn/common/input_output_info.h:31-76, runtime/kernel_exec_context.h
//   EngineImpl / EngineContext            src/ppl/nn/engines/engine_impl.h:43-68, engine_context.h:26-40
//   OptKernel / KernelImpl                src/ppl/nn/runtime/opt_kernel.h:36-49, kernel_impl.h:32-75
#ifndef PPLNN_LLM_HIP_CORE_H_
#define PPLNN_LLM_HIP_CORE_H_

#include <stdio.h>
#include <string.h>

#include <functional>
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

#include "ppl/nn/llm_hip_api.h"

namespace ppl { namespace nn {

using ppl::common::RetCode;

// ---------------------------------------------------------------- logging (LOG(level) << ... as in ppl.common)
enum { LOG_DEBUG = 0, LOG_INFO, LOG_WARNING, LOG_ERROR };
int GetLogLevel();
void SetLogLevel(int);
const std::string& LastErrorMessage(); // last LOG(ERROR) text of the calling thread (for the C test API)
class LogLine final {
public:
    LogLine(int level, const char* file, int line) : level_(level) {
        const char* base = strrchr(file, '/');
        os_ << "[" << (base ? base + 1 : file) << ":" << line << "] ";
    }
    ~LogLine();
    template <typename T>
    LogLine& operator<<(const T& v) {
        os_ << v;
        return *this;
    }

private:
    int level_;
    std::ostringstream os_;
};
#define LOG(level) ::ppl::nn::LogLine(::ppl::nn::LOG_##level, __FILE__, __LINE__)

typedef uint32_t nodeid_t;
typedef uint32_t edgeid_t;
static const uint32_t INVALID_NODEID = UINT32_MAX;
static const uint32_t INVALID_EDGEID = UINT32_MAX;
static const int64_t INVALID_DIM_VALUE = -1;

// ---------------------------------------------------------------- IR
namespace ir {

struct Attr {
    virtual ~Attr() {}
};

struct Node final {
    struct Type final {
        std::string domain;
        std::string name;
        uint64_t version = 0;
    };
    nodeid_t id = INVALID_NODEID;
    std::string name;
    Type type;
    std::vector<edgeid_t> inputs; // INVALID_EDGEID marks an optional input left empty
    std::vector<edgeid_t> outputs;
    nodeid_t GetId() const { return id; }
    const std::string& GetName() const { return name; }
    const Type& GetType() const { return type; }
};

struct Edge final {
    edgeid_t id = INVALID_EDGEID;
    std::string name;
    nodeid_t producer = INVALID_NODEID;
    std::vector<nodeid_t> consumers;
};

struct Shape final {
    ppl::common::datatype_t data_type = ppl::common::DATATYPE_UNKNOWN;
    std::vector<int64_t> dims; // INVALID_DIM_VALUE for symbolic dimensions
};

struct Constant final {
    std::string data; // raw little-endian bytes
};

struct GraphTopo final {
    std::string name;
    std::vector<Node> nodes;
    std::vector<Edge> edges;
    std::vector<edgeid_t> inputs, outputs, constants;
    edgeid_t FindEdge(const std::string& n) const {
        for (auto& e : edges)
            if (e.name == n) return e.id;
        return INVALID_EDGEID;
    }
    edgeid_t AddEdge(const std::string& n) {
        edgeid_t id = FindEdge(n);
        if (id != INVALID_EDGEID) return id;
        Edge e;
        e.id = (edgeid_t)edges.size();
        e.name = n;
        edges.push_back(e);
        return e.id;
    }
};

struct GraphData final {
    std::map<nodeid_t, std::shared_ptr<Attr>> attrs;
    std::map<edgeid_t, Shape> shapes;
    std::map<edgeid_t, Constant> constants;
};

struct Graph final {
    std::shared_ptr<GraphTopo> topo;
    std::shared_ptr<GraphData> data;
};

} // namespace ir

// ---------------------------------------------------------------- registry
namespace utils {

struct VersionRange final {
    uint64_t first = 0, last = 0;
};

template <typename T>
class OpInfoManager final {
public:
    // overlapping ranges for the same (domain, type) -> RC_EXISTS
    RetCode Register(const std::string& domain, const std::string& type, const VersionRange& ver, const T& item) {
        auto& vec = info_[domain][type];
        for (auto& x : vec)
            if (!(ver.last < x.ver.first || x.ver.last < ver.first)) return ppl::common::RC_EXISTS;
        vec.push_back(Item{ver, item});
        return ppl::common::RC_SUCCESS;
    }
    const T* Find(const std::string& domain, const std::string& type, uint64_t version) const {
        auto d = info_.find(domain);
        if (d == info_.end()) return nullptr;
        auto t = d->second.find(type);
        if (t == d->second.end()) return nullptr;
        for (auto& x : t->second)
            if (x.ver.first <= version && version <= x.ver.last) return &x.item;
        return nullptr;
    }
    void Remove(const std::string& domain, const std::string& type) {
        auto d = info_.find(domain);
        if (d != info_.end()) d->second.erase(type);
    }

private:
    struct Item final {
        VersionRange ver;
        T item;
    };
    std::map<std::string, std::map<std::string, std::vector<Item>>> info_;
};

} // namespace utils

// ---------------------------------------------------------------- device + buffers
struct BufferDesc final {
    BufferDesc(void* a = nullptr) : addr(a), desc(0) {}
    void* addr;
    uint64_t desc; // allocation size kept for the manager
};

class Device : public DeviceContext {
public:
    virtual ~Device() {}
    virtual RetCode Realloc(uint64_t bytes, BufferDesc* buffer) = 0;
    RetCode Realloc(const TensorShape& shape, BufferDesc* buffer) {
        return Realloc(shape.CalcBytesIncludingPadding(), buffer);
    }
    virtual void Free(BufferDesc* buffer) = 0;
    virtual RetCode CopyFromHost(BufferDesc* dst, const void* src, uint64_t bytes) const = 0;
    virtual RetCode CopyFromHostAsync(BufferDesc* dst, const void* src, uint64_t bytes) const = 0;
    virtual RetCode CopyToHost(void* dst, const BufferDesc& src, uint64_t bytes) const = 0;
    virtual RetCode CopyToHostAsync(void* dst, const BufferDesc& src, uint64_t bytes) const = 0;
    virtual RetCode Copy(BufferDesc* dst, const BufferDesc& src, uint64_t bytes) const = 0;
    bool IsType(const char* tag) const { return strncmp(GetType().str, tag, 8) == 0; }
};

Device* GetSharedHostDevice(); // process-wide "cpu" device (malloc/free)
class OptKernel;
namespace onnx { class RuntimeBuilder; }
// the op object Preprocess() built for the named node (nullptr before Preprocess or for an unknown name)
OptKernel* FindOpOfBuilder(onnx::RuntimeBuilder* builder, const char* node_name);
class TensorImpl;
// "<tensor name with '/' replaced by '.'>-<dims joined by '_' | scalar | none>-<lower-case type name>.dat"
std::string DumpFileTail(const TensorImpl* tensor);

// ownership rules of src/ppl/nn/common/buffer_info.cc:65-113
class BufferInfo final {
public:
    ~BufferInfo() { FreeBuffer(); }
    void SetDevice(Device* dev) {
        FreeBuffer();
        device_ = dev;
    }
    Device* GetDevice() const { return device_; }
    void SetBuffer(const BufferDesc& buf, Device* dev = nullptr, bool is_owner = false) {
        if (is_buffer_owner_ && device_) device_->Free(&buffer_);
        if (dev) device_ = dev;
        buffer_ = buf;
        is_buffer_owner_ = is_owner;
    }
    RetCode ReallocBuffer(const TensorShape& shape) {
        if (!device_) return ppl::common::RC_PERMISSION_DENIED;
        if (!is_buffer_owner_) buffer_ = BufferDesc(); // a borrowed pointer is dropped, never freed
        auto rc = device_->Realloc(shape, &buffer_);
        if (rc != ppl::common::RC_SUCCESS) return rc;
        is_buffer_owner_ = true;
        return rc;
    }
    void FreeBuffer() {
        if (is_buffer_owner_ && device_) device_->Free(&buffer_);
        buffer_ = BufferDesc();
        is_buffer_owner_ = false;
    }
    BufferDesc& GetBufferDesc() { return buffer_; }
    const BufferDesc& GetBufferDesc() const { return buffer_; }
    bool IsBufferOwner() const { return is_buffer_owner_; }
    // takes over src's buffer, device and ownership; src is left empty
    void MoveFrom(BufferInfo* src) {
        if (src == this) return;
        FreeBuffer();
        buffer_ = src->buffer_;
        device_ = src->device_;
        is_buffer_owner_ = src->is_buffer_owner_;
        src->buffer_ = BufferDesc();
        src->is_buffer_owner_ = false;
    }

private:
    BufferDesc buffer_;
    Device* device_ = nullptr;
    bool is_buffer_owner_ = false;
};

class TensorImpl final : public Tensor {
public:
    TensorImpl(const std::string& name, edgeid_t eid) : name_(name), eid_(eid) {}
    const char* GetName() const override { return name_.c_str(); }
    edgeid_t GetEdgeId() const { return eid_; }
    TensorShape* GetShape() const override { return &shape_; }
    RetCode CopyToHost(void* dst) const override;
    RetCode CopyToHostAsync(void* dst) const override;
    RetCode CopyFromHost(const void* src) override;
    RetCode CopyFromHostAsync(const void* src) override;
    RetCode ConvertToHost(void* dst, const TensorShape& dst_desc) const override;
    RetCode ConvertFromHost(const void* src, const TensorShape& src_desc) override;
    DeviceContext* GetDeviceContext() const override { return info_.GetDevice(); }
    void SetDeviceContext(DeviceContext* ctx) override { info_.SetDevice(static_cast<Device*>(ctx)); }
    void FreeBuffer() override { info_.FreeBuffer(); }
    void SetBufferPtr(void* buf) override { info_.SetBuffer(BufferDesc(buf)); } // non-owning
    void* GetBufferPtr() const override { return info_.GetBufferDesc().addr; }
    template <typename T>
    T* GetBufferPtr() const {
        return static_cast<T*>(info_.GetBufferDesc().addr);
    }
    Device* GetDevice() const { return info_.GetDevice(); }
    void SetDevice(Device* d) { info_.SetDevice(d); }
    // no-op for a non-null pointer the tensor does not own (src/ppl/nn/runtime/tensor_impl.cc:25-32)
    RetCode ReallocBuffer() {
        if (!info_.IsBufferOwner() && info_.GetBufferDesc().addr) return ppl::common::RC_SUCCESS;
        return info_.ReallocBuffer(shape_);
    }
    BufferInfo& GetBufferInfo() { return info_; }
    // in-place ops hand their input's buffer to the output when they are its last consumer
    // (TensorImpl::TransferBufferFrom, used at rotary_position_embedding_kernel.cc:66-76)
    void TransferBufferFrom(TensorImpl* src) { info_.MoveFrom(&src->info_); }

private:
    std::string name_;
    edgeid_t eid_;
    mutable TensorShape shape_;
    BufferInfo info_;
};

// ---------------------------------------------------------------- kernel boundary
class InputOutputInfo {
public:
    void SetNode(const ir::Node* n) { node_ = n; }
    const ir::Node* GetNode() const { return node_; }
    uint32_t GetInputCount() const { return (uint32_t)node_->inputs.size(); }
    uint32_t GetOutputCount() const { return (uint32_t)node_->outputs.size(); }
    template <typename T>
    T* GetInput(uint32_t idx) const {
        if (idx >= node_->inputs.size() || node_->inputs[idx] == INVALID_EDGEID) return nullptr;
        return static_cast<T*>(acquire_(node_->inputs[idx]));
    }
    template <typename T>
    T* GetOutput(uint32_t idx) const {
        if (idx >= node_->outputs.size() || node_->outputs[idx] == INVALID_EDGEID) return nullptr;
        return static_cast<T*>(acquire_(node_->outputs[idx]));
    }
    void SetAcquireFunc(const std::function<TensorImpl*(edgeid_t)>& f) { acquire_ = f; }

protected:
    const ir::Node* node_ = nullptr;
    std::function<TensorImpl*(edgeid_t)> acquire_;
};

class KernelExecContext final : public InputOutputInfo {
public:
    void SetLastConsumerFunc(const std::function<bool(edgeid_t, nodeid_t)>& f) { last_consumer_ = f; }
    bool IsLastConsumerOfInput(uint32_t idx) const {
        return last_consumer_ && last_consumer_(node_->inputs[idx], node_->id);
    }

private:
    std::function<bool(edgeid_t, nodeid_t)> last_consumer_;
};

class EngineContext {
public:
    virtual ~EngineContext() {}
    virtual const char* GetName() const = 0;
    virtual Device* GetDevice() const = 0;
};

class KernelImpl {
public:
    KernelImpl(const ir::Node* node) : node_(node) {}
    virtual ~KernelImpl() {}
    const ir::Node* GetNode() const { return node_; }
    const std::string& GetName() const { return node_->name; }
    const ir::Node::Type& GetType() const { return node_->type; }
    void SetEngineContext(EngineContext* ctx) { engine_context_ = ctx; }
    EngineContext* GetEngineContext() const { return engine_context_; }
    virtual RetCode Reshape(InputOutputInfo*) const = 0;
    virtual RetCode Execute(KernelExecContext*) = 0;
    // microseconds spent in the last Execute (0 when profiling is off); synchronises on the kernel's events
    virtual uint64_t GetExecutionTime() const { return 0; }
    virtual void SetProfilingFlag(bool) {}

private:
    const ir::Node* node_;
    EngineContext* engine_context_ = nullptr;
};

class OptKernel {
public:
    OptKernel(const ir::Node* node) : node_(node) {}
    virtual ~OptKernel() {}
    const ir::Node* GetNode() const { return node_; }
    virtual KernelImpl* CreateKernelImpl() const = 0; // shared, read-only after Init
    // PMX model hooks (src/ppl/nn/runtime/opt_kernel.h: SerializeData / DeserializeData): the op's parameters as a
    // FlatBuffers OpParam blob. Ops without parameters write nothing.
    virtual RetCode SerializeData(std::string* blob) const {
        blob->clear();
        return ppl::common::RC_SUCCESS;
    }
    virtual RetCode DeserializeData(const void*, uint64_t) { return ppl::common::RC_SUCCESS; }

private:
    const ir::Node* node_;
};

struct RuntimePartitionInfo final {
    std::map<edgeid_t, std::unique_ptr<TensorImpl>> constants;
    std::map<nodeid_t, std::unique_ptr<OptKernel>> kernels;
};

class EngineImpl : public Engine {
public:
    EngineImpl(const std::string& name) : name_(name) {}
    const char* GetName() const override final { return name_.c_str(); }
    virtual EngineContext* CreateEngineContext() = 0;
    virtual bool Supports(const ir::Node*) const = 0;
    // must fill info->kernels[node_id] for every node and must not touch graph input/output edges
    virtual RetCode ProcessGraph(ir::Graph*, RuntimePartitionInfo*) = 0;

private:
    const std::string name_;
};

// ---------------------------------------------------------------- ONNX model loading (onnx_parser.cc)
namespace onnx {
// parses a serialized ONNX ModelProto (the subset of fields the reference loader reads) into an ir::Graph; op attributes of
// registered (domain, type) pairs become typed ir::Attr objects in graph->data->attrs
RetCode ParseModel(const char* buf, uint64_t size, ir::Graph* graph);
} // namespace onnx

}} // namespace ppl::nn

#endif
