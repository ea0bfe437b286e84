// Flat C entry points over the C++ engine API, for hosts without a C++ binding (the Python tests use them via ctypes).
// Every function returns a ppl::common::RetCode or a handle (NULL on failure, text in pplnn_hip_last_error()).
#include <cstring>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

#include "arena.h"
#include "core.h"

using namespace ppl::nn;
using namespace ppl::common;

extern "C" {

const char* pplnn_hip_last_error(void) { return LastErrorMessage().c_str(); }
void pplnn_hip_set_log_level(int level) { SetLogLevel(level); }

// ---- engine
void* pplnn_hip_engine_create(uint32_t device_id, uint32_t mm_policy) {
    llm::hip::EngineOptions options;
    options.device_id = device_id;
    options.mm_policy = mm_policy;
    return llm::hip::EngineFactory::Create(options);
}
// every Runtime of the engine enqueues on the caller's stream (EngineOptions::runtime_stream) instead of one of its own
void* pplnn_hip_engine_create_on_stream(uint32_t device_id, uint32_t mm_policy, void* stream) {
    llm::hip::EngineOptions options;
    options.device_id = device_id;
    options.mm_policy = mm_policy;
    options.runtime_stream = stream;
    return llm::hip::EngineFactory::Create(options);
}
const char* pplnn_hip_engine_name(void* e) { return static_cast<Engine*>(e)->GetName(); }
uint32_t pplnn_hip_engine_configure_u32(void* e, uint32_t option, uint32_t value) {
    return static_cast<Engine*>(e)->Configure(option, value);
}
uint32_t pplnn_hip_engine_configure_str(void* e, uint32_t option, const char* value) {
    return static_cast<Engine*>(e)->Configure(option, value);
}
void pplnn_hip_engine_destroy(void* e) { delete static_cast<Engine*>(e); }

// ---- x86 engine (the CPU baseline behind the same builder / runtime calls)
void* pplnn_x86_engine_create(void) { return x86::EngineFactory::Create(x86::EngineOptions()); }
void pplnn_x86_set_num_threads(int n) { x86::SetGlobalOmpNumThreads(n); }
int pplnn_x86_get_num_threads(void) { return x86::GetGlobalOmpNumThreads(); }

// ---- builder
void* pplnn_hip_builder_create(void) { return onnx::RuntimeBuilderFactory::Create(); }
uint32_t pplnn_hip_builder_load_model(void* b, const char* buf, uint64_t len) {
    return static_cast<onnx::RuntimeBuilder*>(b)->LoadModel(buf, len, nullptr);
}
uint32_t pplnn_hip_builder_load_model_file(void* b, const char* path) {
    return static_cast<onnx::RuntimeBuilder*>(b)->LoadModel(path);
}
uint32_t pplnn_hip_builder_set_engine(void* b, void* engine) {
    Engine* engines[1] = {static_cast<Engine*>(engine)};
    onnx::RuntimeBuilder::Resources r;
    r.engines = engines;
    r.engine_num = 1;
    return static_cast<onnx::RuntimeBuilder*>(b)->SetResources(r);
}
uint32_t pplnn_hip_builder_preprocess(void* b) { return static_cast<onnx::RuntimeBuilder*>(b)->Preprocess(); }
void* pplnn_hip_builder_create_runtime(void* b) { return static_cast<onnx::RuntimeBuilder*>(b)->CreateRuntime(); }
void pplnn_hip_builder_destroy(void* b) { delete static_cast<onnx::RuntimeBuilder*>(b); }
// PMX hooks of the op built for a node: its parameters as a FlatBuffers OpParam blob, and back
uint32_t pplnn_hip_builder_serialize_op(void* b, const char* node_name, void* buf, uint64_t cap, uint64_t* size) {
    auto op = FindOpOfBuilder(static_cast<onnx::RuntimeBuilder*>(b), node_name);
    if (!op) {
        LOG(ERROR) << "no op for node[" << node_name << "]";
        return RC_NOT_FOUND;
    }
    std::string blob;
    const RetCode rc = op->SerializeData(&blob);
    if (rc != RC_SUCCESS) return rc;
    *size = blob.size();
    if (blob.size() > cap) return RC_OUT_OF_RANGE;
    memcpy(buf, blob.data(), blob.size());
    return RC_SUCCESS;
}
uint32_t pplnn_hip_builder_deserialize_op(void* b, const char* node_name, const void* buf, uint64_t size) {
    auto op = FindOpOfBuilder(static_cast<onnx::RuntimeBuilder*>(b), node_name);
    if (!op) {
        LOG(ERROR) << "no op for node[" << node_name << "]";
        return RC_NOT_FOUND;
    }
    return op->DeserializeData(buf, size);
}

// ---- runtime
uint32_t pplnn_hip_runtime_input_count(void* r) { return static_cast<Runtime*>(r)->GetInputCount(); }
uint32_t pplnn_hip_runtime_output_count(void* r) { return static_cast<Runtime*>(r)->GetOutputCount(); }
void* pplnn_hip_runtime_input(void* r, uint32_t i) { return static_cast<Runtime*>(r)->GetInputTensor(i); }
void* pplnn_hip_runtime_output(void* r, uint32_t i) { return static_cast<Runtime*>(r)->GetOutputTensor(i); }
uint32_t pplnn_hip_runtime_run(void* r) { return static_cast<Runtime*>(r)->Run(); }
uint32_t pplnn_hip_runtime_run_async(void* r) { return static_cast<Runtime*>(r)->RunAsync(); }
uint32_t pplnn_hip_runtime_synchronize(void* r) { return static_cast<Runtime*>(r)->Synchronize(); }
uint32_t pplnn_hip_runtime_set_profiling(void* r, uint32_t on) {
    return static_cast<Runtime*>(r)->Configure(RUNTIME_CONF_SET_KERNEL_PROFILING_FLAG, on);
}
// writes up to `cap` entries; returns the number of kernels (or 0 with an error recorded)
uint32_t pplnn_hip_runtime_profiling(void* r, uint64_t* micros, uint32_t* counts, uint32_t cap) {
    ProfilingStatistics st;
    if (static_cast<Runtime*>(r)->GetProfilingStatistics(&st) != RC_SUCCESS) return 0;
    for (uint32_t i = 0; i < st.prof_info.size() && i < cap; ++i) {
        micros[i] = st.prof_info[i].exec_microseconds;
        counts[i] = st.prof_info[i].exec_count;
    }
    return (uint32_t)st.prof_info.size();
}
// Step replay, file conventions of tools/pplnn_llm.cc: one file per graph input, comma separated, each named
// "<anything>-<d0_d1_...>-<dtype>.dat" (SetShapedInputsOneByOne, :648-753: shape and type come from the NAME, the
// bytes from the file); outputs go to "<dir>/pplnn_output-<tensor name>.dat" (SaveOutputsOneByOne, :796-822).
uint32_t pplnn_hip_runtime_set_inputs_from_files(void* r, const char* files_csv) {
    auto rt = static_cast<Runtime*>(r);
    std::vector<std::string> files;
    std::string cur;
    for (const char* p = files_csv; ; ++p) {
        if (*p == ',' || *p == 0) {
            if (!cur.empty()) files.push_back(cur);
            cur.clear();
            if (*p == 0) break;
        } else {
            cur.push_back(*p);
        }
    }
    if (files.size() != rt->GetInputCount()) {
        LOG(ERROR) << "input file num[" << files.size() << "] != graph input num[" << rt->GetInputCount() << "]";
        return RC_INVALID_VALUE;
    }
    for (uint32_t c = 0; c < files.size(); ++c) {
        const std::string& path = files[c];
        const size_t slash = path.find_last_of('/');
        const std::string base = slash == std::string::npos ? path : path.substr(slash + 1);
        std::vector<std::string> parts(1);
        for (char ch : base) {
            if (ch == '-') parts.emplace_back();
            else parts.back().push_back(ch);
        }
        if (parts.size() != 3) {
            LOG(ERROR) << "illegal file name format: " << base;
            return RC_INVALID_VALUE;
        }
        const std::string dt_str = parts[2].substr(0, parts[2].find('.'));
        datatype_t dt = DATATYPE_UNKNOWN;
        for (uint32_t t = 0; t < 32; ++t)
            if (dt_str == GetDataTypeStr((datatype_t)t) && dt_str != "unknown") dt = (datatype_t)t;
        if (dt == DATATYPE_UNKNOWN) {
            LOG(ERROR) << "cannot find data type[" << dt_str << "] in input file[" << base << "]";
            return RC_INVALID_VALUE;
        }
        std::vector<int64_t> dims;
        bool scalar = parts[1] == "scalar";
        if (!scalar && parts[1] != "none") {
            std::string d;
            for (size_t i = 0; i <= parts[1].size(); ++i) {
                if (i == parts[1].size() || parts[1][i] == '_') {
                    if (d.empty()) {
                        LOG(ERROR) << "illegal dim format.";
                        return RC_INVALID_VALUE;
                    }
                    dims.push_back(atol(d.c_str()));
                    d.clear();
                } else {
                    d.push_back(parts[1][i]);
                }
            }
        }
        auto t = rt->GetInputTensor(c);
        t->GetShape()->SetDataType(dt);
        if (scalar) t->GetShape()->ReshapeAsScalar();
        else t->GetShape()->Reshape(dims.data(), (uint32_t)dims.size());
        const uint64_t bytes = t->GetShape()->CalcBytesIncludingPadding();
        if (bytes == 0) continue;
        std::ifstream f(path, std::ios::binary);
        if (!f) {
            LOG(ERROR) << "mapping file[" << path << "] failed.";
            return RC_NOT_FOUND;
        }
        std::string data((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
        if (data.size() < bytes) {
            LOG(ERROR) << "input file[" << base << "] size(" << data.size() << ") is less than tensor[" << t->GetName()
                       << "] size(" << bytes << ")";
            return RC_INVALID_VALUE;
        }
        const RetCode rc = t->ConvertFromHost(data.data(), *t->GetShape());
        if (rc != RC_SUCCESS) {
            LOG(ERROR) << "set input[" << t->GetName() << "] failed: " << GetRetCodeStr(rc);
            return rc;
        }
    }
    return RC_SUCCESS;
}
uint32_t pplnn_hip_runtime_save_outputs(void* r, const char* dir) {
    auto rt = static_cast<Runtime*>(r);
    for (uint32_t c = 0; c < rt->GetOutputCount(); ++c) {
        auto t = rt->GetOutputTensor(c);
        std::vector<char> buffer(t->GetShape()->CalcBytesIncludingPadding());
        const RetCode rc = t->ConvertToHost(buffer.data(), *t->GetShape());
        if (rc != RC_SUCCESS) {
            LOG(ERROR) << "convert data of tensor[" << t->GetName() << "] failed: " << GetRetCodeStr(rc);
            return rc;
        }
        const std::string file = std::string(dir) + "/pplnn_output-" + t->GetName() + ".dat";
        std::ofstream ofs(file, std::ios_base::out | std::ios_base::binary | std::ios_base::trunc);
        if (!ofs.is_open()) {
            LOG(ERROR) << "open output file[" << file << "]";
            return RC_OTHER_ERROR;
        }
        ofs.write(buffer.data(), buffer.size());
    }
    return RC_SUCCESS;
}
void pplnn_hip_runtime_destroy(void* r) { delete static_cast<Runtime*>(r); }

// ---- tensor
const char* pplnn_hip_tensor_name(void* t) { return static_cast<Tensor*>(t)->GetName(); }
void pplnn_hip_tensor_reshape(void* t, const int64_t* dims, uint32_t n) {
    if (n == 0) static_cast<Tensor*>(t)->GetShape()->ReshapeAsScalar();
    else static_cast<Tensor*>(t)->GetShape()->Reshape(dims, n);
}
uint32_t pplnn_hip_tensor_dims(void* t, int64_t* dims, uint32_t cap) {
    auto s = static_cast<Tensor*>(t)->GetShape();
    for (uint32_t i = 0; i < s->GetDimCount() && i < cap; ++i) dims[i] = s->GetDim(i);
    return s->GetDimCount();
}
uint32_t pplnn_hip_tensor_dtype(void* t) { return static_cast<Tensor*>(t)->GetShape()->GetDataType(); }
void pplnn_hip_tensor_set_buffer_ptr(void* t, void* p) { static_cast<Tensor*>(t)->SetBufferPtr(p); }
void* pplnn_hip_tensor_buffer_ptr(void* t) { return static_cast<Tensor*>(t)->GetBufferPtr(); }
uint32_t pplnn_hip_tensor_copy_from_host(void* t, const void* src) { return static_cast<Tensor*>(t)->CopyFromHost(src); }
uint32_t pplnn_hip_tensor_copy_to_host(void* t, void* dst) { return static_cast<Tensor*>(t)->CopyToHost(dst); }
// places the tensor on the host device, like `Tensor::SetDeviceContext(host_device)` for the scalar inputs
void pplnn_hip_tensor_use_host_device(void* t) { static_cast<Tensor*>(t)->SetDeviceContext(GetSharedHostDevice()); }

// ---- self-checks of host components that need no GPU
// registering two overlapping version ranges for the same op must give RC_EXISTS (utils/op_info_manager.h:49-71)
uint32_t pplnn_hip_selftest_registry(void) {
    utils::OpInfoManager<int> m;
    if (m.Register("d", "T", utils::VersionRange{1, 5}, 1) != RC_SUCCESS) return RC_OTHER_ERROR;
    if (m.Register("d", "T", utils::VersionRange{6, 9}, 2) != RC_SUCCESS) return RC_OTHER_ERROR;
    if (m.Register("d", "T", utils::VersionRange{5, 6}, 3) != RC_EXISTS) return RC_OTHER_ERROR;
    if (!m.Find("d", "T", 7) || *m.Find("d", "T", 7) != 2 || m.Find("d", "T", 10) || m.Find("x", "T", 1)) return RC_OTHER_ERROR;
    return RC_EXISTS;
}

void* pplnn_hip_arena_create_host(uint64_t alignment, uint64_t block_bytes) {
    return new utils::ArenaBufferManager([](uint64_t n) { return malloc(n); }, [](void* p) { free(p); }, alignment, block_bytes);
}
// mm_policy: MM_PLAIN / MM_COMPACT / MM_BEST_FIT of the llm_hip engine options
void* pplnn_hip_arena_create_host_with_policy(uint64_t alignment, uint64_t block_bytes, uint32_t mm_policy) {
    const auto policy = mm_policy == llm::hip::MM_PLAIN     ? utils::ArenaBufferManager::kPlain
                        : mm_policy == llm::hip::MM_COMPACT ? utils::ArenaBufferManager::kCompact
                                                            : utils::ArenaBufferManager::kBestFit;
    return new utils::ArenaBufferManager([](uint64_t n) { return malloc(n); }, [](void* p) { free(p); }, alignment,
                                         block_bytes, policy);
}
uint32_t pplnn_hip_arena_alloc(void* a, uint64_t bytes, void** addr, uint64_t* desc) {
    BufferDesc b;
    auto rc = static_cast<utils::ArenaBufferManager*>(a)->Alloc(bytes, &b);
    *addr = b.addr;
    *desc = b.desc;
    return rc;
}
void pplnn_hip_arena_free(void* a, void* addr) {
    BufferDesc b(addr);
    static_cast<utils::ArenaBufferManager*>(a)->Free(&b);
}
uint64_t pplnn_hip_arena_buffered_bytes(void* a) { return static_cast<utils::ArenaBufferManager*>(a)->GetBufferedBytes(); }
uint64_t pplnn_hip_arena_used_bytes(void* a) { return static_cast<utils::ArenaBufferManager*>(a)->GetUsedBytes(); }
void pplnn_hip_arena_destroy(void* a) { delete static_cast<utils::ArenaBufferManager*>(a); }

} // extern "C"
