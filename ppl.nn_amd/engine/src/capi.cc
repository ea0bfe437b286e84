// Flat C entry points over the C++ engine API, for hosts without a C++ binding (the Python tests use them via ctypes).
// Every function returns a ppl::common::RetCode or a handle (NULL on failure, text in pplnn_hip_last_error()).
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
const char* pplnn_hip_engine_name(void* e) { return static_cast<Engine*>(e)->GetName(); }
uint32_t pplnn_hip_engine_configure_u32(void* e, uint32_t option, uint32_t value) {
    return static_cast<Engine*>(e)->Configure(option, value);
}
void pplnn_hip_engine_destroy(void* e) { delete static_cast<Engine*>(e); }

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

// ---- runtime
uint32_t pplnn_hip_runtime_input_count(void* r) { return static_cast<Runtime*>(r)->GetInputCount(); }
uint32_t pplnn_hip_runtime_output_count(void* r) { return static_cast<Runtime*>(r)->GetOutputCount(); }
void* pplnn_hip_runtime_input(void* r, uint32_t i) { return static_cast<Runtime*>(r)->GetInputTensor(i); }
void* pplnn_hip_runtime_output(void* r, uint32_t i) { return static_cast<Runtime*>(r)->GetOutputTensor(i); }
uint32_t pplnn_hip_runtime_run(void* r) { return static_cast<Runtime*>(r)->Run(); }
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
