// Common helpers, the host device, TensorImpl, the ONNX RuntimeBuilder and the sequential runtime. Restates
//   RuntimeBuilderImpl    src/ppl/nn/models/onnx/runtime_builder_impl.cc:55-145
//   ProcessGraph          src/ppl/nn/optimizers/utils.cc:366-420 (one engine, one partition on this path)
//   RuntimeAuxInfo        src/ppl/nn/runtime/runtime_aux_info.cc:27-38 (topological order, last consumers: runtime/utils.cc:26-150)
//   RuntimeImpl           src/ppl/nn/runtime/runtime_impl.cc:57-327, 450-515
//   SequentialScheduler   src/ppl/nn/runtime/sequential_scheduler.cc:31-179
//   Profiler              src/ppl/nn/runtime/profiler.cc:31-37
#include <stdlib.h>

#include <fstream>
#include <mutex>

#include "core.h"

using namespace ppl::common;

namespace ppl { namespace common {

const char* GetRetCodeStr(RetCode rc) {
    static const char* names[] = {"success",       "other error",       "unsupported",         "out of memory",
                                  "invalid value", "exists",            "not found",           "permission denied",
                                  "host memory error", "device memory error", "device runtime error", "out of range",
                                  "internal error"};
    return rc < sizeof(names) / sizeof(names[0]) ? names[rc] : "unknown";
}

uint32_t GetSizeOfDataType(datatype_t t) {
    switch (t) {
        case DATATYPE_UINT8: case DATATYPE_INT8: case DATATYPE_BOOL: return 1;
        case DATATYPE_UINT16: case DATATYPE_INT16: case DATATYPE_FLOAT16: case DATATYPE_BFLOAT16: return 2;
        case DATATYPE_UINT32: case DATATYPE_INT32: case DATATYPE_FLOAT32: return 4;
        case DATATYPE_UINT64: case DATATYPE_INT64: case DATATYPE_FLOAT64: return 8;
        default: return 0;
    }
}

const char* GetDataTypeStr(datatype_t t) {
    static const char* names[] = {"unknown", "uint8", "uint16", "uint32", "uint64", "fp16", "fp32", "fp64",
                                  "bf16",    "int4b", "int8",   "int16",  "int32",  "int64", "bool"};
    return t < sizeof(names) / sizeof(names[0]) ? names[t] : "unknown";
}

}} // namespace ppl::common

namespace ppl { namespace nn {

// ---------------------------------------------------------------- logging
static int g_log_level = LOG_WARNING;
static thread_local std::string g_last_error;
int GetLogLevel() { return g_log_level; }
void SetLogLevel(int l) { g_log_level = l; }
const std::string& LastErrorMessage() { return g_last_error; }
LogLine::~LogLine() {
    if (level_ == LOG_ERROR) { // every layer logs as the error propagates: keep the innermost few lines too
        static thread_local std::vector<std::string> recent;
        recent.push_back(os_.str());
        if (recent.size() > 4) recent.erase(recent.begin());
        g_last_error.clear();
        for (auto& r : recent) g_last_error += (g_last_error.empty() ? "" : " | ") + r;
    }
    if (level_ >= g_log_level) {
        static const char* tags[] = {"DEBUG", "INFO", "WARNING", "ERROR"};
        fprintf(stderr, "[%s]%s\n", tags[level_], os_.str().c_str());
    }
}

// ---------------------------------------------------------------- host device
namespace {
class HostDevice final : public Device {
public:
    const Type& GetType() const override {
        static const Type t = {{'c', 'p', 'u', 0, 0, 0, 0, 0}};
        return t;
    }
    RetCode Synchronize() override { return RC_SUCCESS; }
    RetCode Configure(uint32_t, ...) override { return RC_UNSUPPORTED; }
    RetCode Realloc(uint64_t bytes, BufferDesc* buffer) override {
        if (buffer->addr && buffer->desc >= bytes) return RC_SUCCESS;
        if (buffer->addr) free(buffer->addr);
        buffer->addr = nullptr;
        buffer->desc = 0;
        if (bytes == 0) return RC_SUCCESS;
        if (posix_memalign(&buffer->addr, 64, (bytes + 63) / 64 * 64)) {
            buffer->addr = nullptr;
            return RC_OUT_OF_MEMORY;
        }
        buffer->desc = bytes;
        return RC_SUCCESS;
    }
    void Free(BufferDesc* buffer) override {
        free(buffer->addr);
        buffer->addr = nullptr;
        buffer->desc = 0;
    }
    RetCode CopyFromHost(BufferDesc* dst, const void* src, uint64_t bytes) const override {
        memcpy(dst->addr, src, bytes);
        return RC_SUCCESS;
    }
    RetCode CopyFromHostAsync(BufferDesc* dst, const void* src, uint64_t bytes) const override {
        return CopyFromHost(dst, src, bytes);
    }
    RetCode CopyToHost(void* dst, const BufferDesc& src, uint64_t bytes) const override {
        memcpy(dst, src.addr, bytes);
        return RC_SUCCESS;
    }
    RetCode CopyToHostAsync(void* dst, const BufferDesc& src, uint64_t bytes) const override {
        return CopyToHost(dst, src, bytes);
    }
    RetCode Copy(BufferDesc* dst, const BufferDesc& src, uint64_t bytes) const override {
        memcpy(dst->addr, src.addr, bytes);
        return RC_SUCCESS;
    }
};
} // namespace

Device* GetSharedHostDevice() {
    static HostDevice dev;
    return &dev;
}

// ---------------------------------------------------------------- TensorImpl
RetCode TensorImpl::CopyToHost(void* dst) const {
    if (!info_.GetDevice() || !info_.GetBufferDesc().addr) return RC_NOT_FOUND;
    return info_.GetDevice()->CopyToHost(dst, info_.GetBufferDesc(), shape_.CalcBytesIncludingPadding());
}
RetCode TensorImpl::CopyToHostAsync(void* dst) const {
    if (!info_.GetDevice() || !info_.GetBufferDesc().addr) return RC_NOT_FOUND;
    return info_.GetDevice()->CopyToHostAsync(dst, info_.GetBufferDesc(), shape_.CalcBytesIncludingPadding());
}
RetCode TensorImpl::CopyFromHost(const void* src) {
    auto rc = ReallocBuffer();
    if (rc != RC_SUCCESS) return rc;
    return info_.GetDevice()->CopyFromHost(&info_.GetBufferDesc(), src, shape_.CalcBytesIncludingPadding());
}
RetCode TensorImpl::CopyFromHostAsync(const void* src) {
    auto rc = ReallocBuffer();
    if (rc != RC_SUCCESS) return rc;
    return info_.GetDevice()->CopyFromHostAsync(&info_.GetBufferDesc(), src, shape_.CalcBytesIncludingPadding());
}
// only identical type + format, like the reference device (llm_cuda_device.cc:224-244)
RetCode TensorImpl::ConvertToHost(void* dst, const TensorShape& dst_desc) const {
    if (dst_desc.GetDataType() != shape_.GetDataType()) {
        LOG(ERROR) << "only support same datatype conversion";
        return RC_UNSUPPORTED;
    }
    return CopyToHost(dst);
}
RetCode TensorImpl::ConvertFromHost(const void* src, const TensorShape& src_desc) {
    if (src_desc.GetDataType() != shape_.GetDataType()) {
        LOG(ERROR) << "only support same datatype conversion";
        return RC_UNSUPPORTED;
    }
    return CopyFromHost(src);
}

// ---------------------------------------------------------------- graph info shared by all runtimes of a builder
struct RuntimeGraphInfo final {
    ir::Graph graph;
    EngineImpl* engine = nullptr;
    RuntimePartitionInfo partition;
    std::vector<nodeid_t> sorted_nodes;
    std::map<edgeid_t, nodeid_t> edge_last_consumer; // edges that may be released, and after which node
};

static RetCode TopologicalSort(const ir::GraphTopo& topo, std::vector<nodeid_t>* order) {
    std::vector<uint32_t> pending(topo.nodes.size(), 0);
    for (auto& n : topo.nodes)
        for (auto e : n.inputs)
            if (e != INVALID_EDGEID && topo.edges[e].producer != INVALID_NODEID) ++pending[n.id];
    std::vector<nodeid_t> ready;
    for (auto& n : topo.nodes)
        if (!pending[n.id]) ready.push_back(n.id);
    while (!ready.empty()) {
        const nodeid_t nid = ready.front();
        ready.erase(ready.begin());
        order->push_back(nid);
        for (auto e : topo.nodes[nid].outputs) {
            if (e == INVALID_EDGEID) continue;
            for (auto c : topo.edges[e].consumers)
                if (--pending[c] == 0) ready.push_back(c);
        }
    }
    if (order->size() != topo.nodes.size()) {
        LOG(ERROR) << "graph has a cycle";
        return RC_INVALID_VALUE;
    }
    return RC_SUCCESS;
}

// ---------------------------------------------------------------- runtime
namespace {

class RuntimeImpl final : public Runtime {
public:
    ~RuntimeImpl() {
        kernels_.clear();
        tensors_.clear(); // tensors free their buffers on devices owned by the engine context, so this goes first
        engine_ctx_.reset();
    }
    RetCode Init(const std::shared_ptr<RuntimeGraphInfo>& info) {
        info_ = info;
        engine_ctx_.reset(info->engine->CreateEngineContext());
        if (!engine_ctx_) {
            LOG(ERROR) << "create engine context of engine[" << info->engine->GetName() << "] failed";
            return RC_OTHER_ERROR;
        }
        auto topo = info->graph.topo.get();
        for (auto nid : info->sorted_nodes) {
            auto it = info->partition.kernels.find(nid);
            if (it == info->partition.kernels.end()) return RC_NOT_FOUND;
            std::unique_ptr<KernelImpl> k(it->second->CreateKernelImpl());
            if (!k) {
                LOG(ERROR) << "create kernel[" << topo->nodes[nid].name << "] failed";
                return RC_OUT_OF_MEMORY;
            }
            k->SetEngineContext(engine_ctx_.get());
            kernels_[nid] = std::move(k);
        }
        // reserved tensors: graph inputs take the device of their first consumer's engine, outputs of their producer
        // (runtime_impl.cc:81-173) -- one engine here, so all of them start on its device
        auto make = [&](edgeid_t eid) -> TensorImpl* {
            auto& t = tensors_[eid];
            if (!t) {
                t.reset(new TensorImpl(topo->edges[eid].name, eid));
                t->SetDevice(engine_ctx_->GetDevice());
                auto s = info->graph.data->shapes.find(eid);
                if (s != info->graph.data->shapes.end()) {
                    t->GetShape()->SetDataType(s->second.data_type);
                    std::vector<int64_t> dims = s->second.dims;
                    if (dims.empty()) t->GetShape()->ReshapeAsScalar();
                    else t->GetShape()->Reshape(dims);
                }
            }
            return t.get();
        };
        for (auto e : topo->inputs) inputs_.push_back(make(e));
        for (auto e : topo->outputs) outputs_.push_back(make(e));
        for (auto e : topo->constants) {
            auto t = make(e);
            auto& c = info->graph.data->constants[e];
            if (c.data.size() < t->GetShape()->CalcBytesIncludingPadding()) { // dims promise more than the payload holds
                LOG(ERROR) << "initializer[" << t->GetName() << "] holds " << c.data.size() << " bytes, its shape needs "
                           << t->GetShape()->CalcBytesIncludingPadding();
                return RC_INVALID_VALUE;
            }
            auto rc = t->CopyFromHost(c.data.data());
            if (rc != RC_SUCCESS) return rc;
        }
        return RC_SUCCESS;
    }
    RetCode Configure(uint32_t option, ...) override {
        va_list args;
        va_start(args, option);
        RetCode rc = RC_SUCCESS;
        if (option == RUNTIME_CONF_SET_KERNEL_PROFILING_FLAG) {
            profiling_ = va_arg(args, uint32_t) ? true : false;
            for (auto& k : kernels_) k.second->SetProfilingFlag(profiling_);
            if (profiling_) stats_.clear();
        } else if (option == RUNTIME_CONF_INFER_SHAPES) {
            rc = InferShapes();
        } else {
            LOG(ERROR) << "invalid option[" << option << "] >= [" << (uint32_t)RUNTIME_CONF_MAX << "]";
            rc = RC_INVALID_VALUE;
        }
        va_end(args);
        return rc;
    }
    uint32_t GetInputCount() const override { return (uint32_t)inputs_.size(); }
    Tensor* GetInputTensor(uint32_t idx) const override { return idx < inputs_.size() ? inputs_[idx] : nullptr; }
    uint32_t GetOutputCount() const override { return (uint32_t)outputs_.size(); }
    Tensor* GetOutputTensor(uint32_t idx) const override { return idx < outputs_.size() ? outputs_[idx] : nullptr; }
    uint32_t GetDeviceContextCount() const override { return 1; }
    DeviceContext* GetDeviceContext(uint32_t idx) const override { return idx == 0 ? engine_ctx_->GetDevice() : nullptr; }
    Tensor* GetTensor(const char* name) const override {
        for (auto& t : tensors_)
            if (t.second && !strcmp(t.second->GetName(), name)) return t.second.get();
        return nullptr;
    }
    RetCode RunAsync() override { return ForEach(true); }
    RetCode Synchronize() override { return engine_ctx_->GetDevice()->Synchronize(); }
    RetCode Run() override { // runtime_impl.cc:320-327: synchronises even when a kernel failed
        auto rc = RunAsync();
        auto rc2 = Synchronize();
        return rc != RC_SUCCESS ? rc : rc2;
    }
    RetCode GetProfilingStatistics(ProfilingStatistics* stat) const override {
        if (!profiling_) {
            LOG(ERROR) << "this version does not support profiling unless RUNTIME_CONF_SET_KERNEL_PROFILING_FLAG is set";
            return RC_UNSUPPORTED;
        }
        stat->prof_info.clear();
        for (auto nid : info_->sorted_nodes) {
            auto& n = info_->graph.topo->nodes[nid];
            ProfilingStatistics::KernelProfilingInfo k;
            k.kernel_name = n.name;
            k.kernel_type = n.type.domain.empty() ? n.type.name : n.type.domain + "." + n.type.name;
            auto it = stats_.find(nid);
            if (it != stats_.end()) {
                k.exec_microseconds = it->second.first;
                k.exec_count = it->second.second;
            }
            stat->prof_info.push_back(k);
        }
        return RC_SUCCESS;
    }

private:
    TensorImpl* Acquire(edgeid_t eid) {
        auto& t = tensors_[eid];
        if (!t) { // intermediate tensors are created lazily on first use (sequential_scheduler.cc:31-87)
            t.reset(new TensorImpl(info_->graph.topo->edges[eid].name, eid));
            t->SetDevice(engine_ctx_->GetDevice());
        }
        return t.get();
    }
    RetCode InferShapes() {
        InputOutputInfo io;
        io.SetAcquireFunc([this](edgeid_t e) { return Acquire(e); });
        for (auto nid : info_->sorted_nodes) {
            io.SetNode(&info_->graph.topo->nodes[nid]);
            auto rc = kernels_[nid]->Reshape(&io);
            if (rc != RC_SUCCESS) return rc;
        }
        return RC_SUCCESS;
    }
    RetCode ForEach(bool) {
        KernelExecContext ctx;
        ctx.SetAcquireFunc([this](edgeid_t e) { return Acquire(e); });
        ctx.SetLastConsumerFunc([this](edgeid_t e, nodeid_t n) {
            auto it = info_->edge_last_consumer.find(e);
            return it != info_->edge_last_consumer.end() && it->second == n;
        });
        for (auto nid : info_->sorted_nodes) {
            auto& node = info_->graph.topo->nodes[nid];
            ctx.SetNode(&node);
            auto kernel = kernels_[nid].get();
            auto rc = kernel->Execute(&ctx);
            if (rc != RC_SUCCESS) {
                LOG(ERROR) << "exec kernel[" << node.name << "] of type[" << node.type.domain << ":" << node.type.name
                           << ":" << node.type.version << "] failed: " << GetRetCodeStr(rc);
                return rc;
            }
            if (profiling_) {
                auto& s = stats_[nid];
                s.first += kernel->GetExecutionTime();
                s.second += 1;
            }
            // release intermediate inputs after their last consumer
            for (auto e : node.inputs) {
                if (e == INVALID_EDGEID) continue;
                auto it = info_->edge_last_consumer.find(e);
                if (it != info_->edge_last_consumer.end() && it->second == nid) {
                    auto t = tensors_.find(e);
                    if (t != tensors_.end() && t->second) t->second->FreeBuffer();
                }
            }
        }
        return RC_SUCCESS;
    }

    std::shared_ptr<RuntimeGraphInfo> info_;
    std::unique_ptr<EngineContext> engine_ctx_;
    std::map<nodeid_t, std::unique_ptr<KernelImpl>> kernels_;
    std::map<edgeid_t, std::unique_ptr<TensorImpl>> tensors_;
    std::vector<TensorImpl*> inputs_, outputs_;
    bool profiling_ = false;
    std::map<nodeid_t, std::pair<uint64_t, uint32_t>> stats_;
};

class RuntimeBuilderImpl final : public onnx::RuntimeBuilder {
public:
    RetCode LoadModel(const char* model_file) override {
        std::ifstream f(model_file, std::ios::binary);
        if (!f) {
            LOG(ERROR) << "open model file[" << model_file << "] failed";
            return RC_NOT_FOUND;
        }
        std::string buf((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
        return LoadModel(buf.data(), buf.size(), nullptr);
    }
    RetCode LoadModel(const char* model_buf, uint64_t buf_len, const char*) override {
        info_ = std::make_shared<RuntimeGraphInfo>();
        auto rc = onnx::ParseModel(model_buf, buf_len, &info_->graph);
        if (rc != RC_SUCCESS) {
            LOG(ERROR) << "parse graph failed: " << GetRetCodeStr(rc);
            info_.reset();
        }
        return rc;
    }
    RetCode SetResources(const Resources& r) override {
        if (r.engine_num == 0 || !r.engines) {
            LOG(ERROR) << "no engine specified";
            return RC_INVALID_VALUE;
        }
        engines_.assign(r.engines, r.engines + r.engine_num);
        return RC_SUCCESS;
    }
    RetCode Preprocess() override {
        if (!info_) {
            LOG(ERROR) << "no model loaded";
            return RC_INVALID_VALUE;
        }
        if (engines_.empty()) {
            LOG(ERROR) << "SetResources() was not called";
            return RC_INVALID_VALUE;
        }
        // partition: every node must be supported by one of the engines; this path has a single partition
        auto topo = info_->graph.topo.get();
        EngineImpl* chosen = nullptr;
        for (auto& node : topo->nodes) {
            EngineImpl* found = nullptr;
            for (auto e : engines_) {
                auto impl = static_cast<EngineImpl*>(e);
                if (impl->Supports(&node)) {
                    found = impl;
                    break;
                }
            }
            if (!found) {
                LOG(ERROR) << "op[" << node.name << "] with type[" << node.type.domain << ":" << node.type.name << ":"
                           << node.type.version << "] is not supported by any engine";
                return RC_UNSUPPORTED;
            }
            if (chosen && chosen != found) {
                LOG(ERROR) << "graphs spanning several engines are not supported";
                return RC_UNSUPPORTED;
            }
            chosen = found;
        }
        if (!chosen) chosen = static_cast<EngineImpl*>(engines_[0]);
        info_->engine = chosen;
        auto rc = chosen->ProcessGraph(&info_->graph, &info_->partition);
        if (rc != RC_SUCCESS) {
            LOG(ERROR) << "process graph by engine[" << chosen->GetName() << "] failed: " << GetRetCodeStr(rc);
            return rc;
        }
        rc = TopologicalSort(*topo, &info_->sorted_nodes);
        if (rc != RC_SUCCESS) return rc;
        // last consumers of intermediate edges; inputs, outputs and constants are never released
        std::vector<uint32_t> position(topo->nodes.size());
        for (uint32_t i = 0; i < info_->sorted_nodes.size(); ++i) position[info_->sorted_nodes[i]] = i;
        auto reserved = [&](edgeid_t e) {
            for (auto x : topo->inputs) if (x == e) return true;
            for (auto x : topo->outputs) if (x == e) return true;
            for (auto x : topo->constants) if (x == e) return true;
            return false;
        };
        for (auto& e : topo->edges) {
            if (reserved(e.id) || e.consumers.empty()) continue;
            nodeid_t last = e.consumers[0];
            for (auto c : e.consumers)
                if (position[c] > position[last]) last = c;
            info_->edge_last_consumer[e.id] = last;
        }
        preprocessed_ = true;
        return RC_SUCCESS;
    }
    Runtime* CreateRuntime() const override {
        if (!preprocessed_) {
            LOG(ERROR) << "Preprocess() was not called";
            return nullptr;
        }
        auto rt = new RuntimeImpl();
        auto rc = rt->Init(info_);
        if (rc != RC_SUCCESS) {
            LOG(ERROR) << "init runtime failed: " << GetRetCodeStr(rc);
            delete rt;
            return nullptr;
        }
        return rt;
    }

    // the op object built for a node by Preprocess(), by node name
    OptKernel* FindOp(const char* node_name) const {
        if (!preprocessed_) return nullptr;
        for (auto& node : info_->graph.topo->nodes) {
            if (node.name != node_name) continue;
            auto it = info_->partition.kernels.find(node.id);
            return it == info_->partition.kernels.end() ? nullptr : it->second.get();
        }
        return nullptr;
    }

private:
    std::shared_ptr<RuntimeGraphInfo> info_;
    std::vector<Engine*> engines_;
    bool preprocessed_ = false;
};

} // namespace

std::string DumpFileTail(const TensorImpl* tensor) {
    auto shape = tensor->GetShape();
    std::string name = tensor->GetName();
    for (auto& c : name)
        if (c == '/') c = '.';
    std::string dims;
    if (shape->IsScalar()) {
        dims = "scalar";
    } else if (shape->GetRealDimCount() == 0) {
        dims = "none";
    } else {
        dims = std::to_string(shape->GetDim(0));
        for (uint32_t i = 1; i < shape->GetDimCount(); ++i) dims += "_" + std::to_string(shape->GetDim(i));
    }
    std::string dt = ppl::common::GetDataTypeStr(shape->GetDataType());
    for (auto& c : dt) c = (char)tolower(c);
    return name + "-" + dims + "-" + dt + ".dat";
}

OptKernel* FindOpOfBuilder(onnx::RuntimeBuilder* builder, const char* node_name) {
    return static_cast<RuntimeBuilderImpl*>(builder)->FindOp(node_name);
}

onnx::RuntimeBuilder* onnx::RuntimeBuilderFactory::Create() {
    return new RuntimeBuilderImpl();
}

}} // namespace ppl::nn
