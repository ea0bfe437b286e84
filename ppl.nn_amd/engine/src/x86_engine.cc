// The x86 engine for the attention subgraph the CPU baseline runs: ONNX MatMul / Mul / Add / Softmax / Transpose in
// fp32 NDARRAY behind the same engine / op / kernel boundary as the llm_hip engine, with the reference wrappers'
// semantics (the arithmetic of the reference lives in its un-vendored ppl.kernel.cpu; these kernels are this build's own):
//   engine + options   src/ppl/nn/engines/x86/engine.cc, include/ppl/nn/engines/x86/{engine_options.h:26-30, options.h:26-63}
//   op registration    src/ppl/nn/engines/x86/optimizer/x86_ops.cc:146,194,199,232,246 (same version ranges)
//   MatMul             src/ppl/nn/engines/x86/kernels/onnx/matmul_kernel.cc:24-57 (fp32 NDARRAY only), shapes by
//                      src/ppl/nn/oputils/onnx/reshape_matmul.cc:26-49 (numpy batch broadcasting)
//   Add / Mul          src/ppl/nn/engines/x86/kernels/onnx/add_kernel.cc:27-91 (in-place when the input dies here)
//   Softmax            src/ppl/nn/engines/x86/kernels/onnx/softmax_kernel.cc:24-62 (opset < 13: 2-D coercion at `axis`)
//   Transpose          src/ppl/nn/oputils/onnx/reshape_transpose.cc:26-44
//   thread count       src/ppl/nn/engines/x86/... SetGlobalOmpNumThreads, used at tools/pplnn.cc:377-380
#include <math.h>
#include <omp.h>

#include <algorithm>
#include <chrono>
#include <mutex>

#include "params.h"

using namespace ppl::common;

namespace ppl { namespace nn { namespace x86 {

struct EngineConfig final {
    bool enable_graph_fusion = true;
    bool enable_tensor_debug = false;
    std::string debug_data_dir = ".";
};

class X86EngineContext final : public EngineContext {
public:
    const char* GetName() const override { return "x86"; }
    Device* GetDevice() const override { return GetSharedHostDevice(); }
};

// ---------------------------------------------------------------- kernel base
class X86Kernel : public KernelImpl {
public:
    X86Kernel(const ir::Node* node) : KernelImpl(node) {}
    RetCode Execute(KernelExecContext* ctx) override final {
        const auto t0 = std::chrono::steady_clock::now();
        auto rc = Reshape(ctx); // shapes follow the inputs of this run (kernel.cc: BeforeExecute)
        if (rc == RC_SUCCESS) rc = DoExecute(ctx);
        if (profiling_)
            micros_ = (uint64_t)std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count();
        return rc;
    }
    uint64_t GetExecutionTime() const override { return profiling_ ? micros_ : 0; }
    void SetProfilingFlag(bool on) override { profiling_ = on; }

protected:
    virtual RetCode DoExecute(KernelExecContext*) = 0;
    static RetCode ReallocOnHost(TensorImpl* t) {
        if (t->GetDevice() != GetSharedHostDevice()) t->SetDevice(GetSharedHostDevice());
        auto rc = t->ReallocBuffer();
        if (rc != RC_SUCCESS) LOG(ERROR) << "ReallocBuffer for tensor[" << t->GetName() << "] failed: " << GetRetCodeStr(rc);
        return rc;
    }
    static bool IsFp32Ndarray(const TensorImpl* t) {
        return t->GetShape()->GetDataType() == DATATYPE_FLOAT32 && t->GetShape()->GetDataFormat() == DATAFORMAT_NDARRAY;
    }

private:
    bool profiling_ = false;
    uint64_t micros_ = 0;
};

#define X86_REQUIRED_INPUT(var, idx)                          \
    auto var = ctx->GetInput<TensorImpl>(idx);                \
    if (!var) {                                               \
        LOG(ERROR) << "Input \"" << #var << "\" is required."; \
        return RC_NOT_FOUND;                                  \
    }
#define X86_REQUIRED_OUTPUT(var, idx)                          \
    auto var = ctx->GetOutput<TensorImpl>(idx);                \
    if (!var) {                                                \
        LOG(ERROR) << "Output \"" << #var << "\" is required."; \
        return RC_NOT_FOUND;                                   \
    }

static std::vector<int64_t> DimsOf(const TensorShape& s) {
    if (s.IsScalar()) return {};
    return std::vector<int64_t>(s.GetDims(), s.GetDims() + s.GetDimCount());
}
static void SetDims(TensorShape* s, const std::vector<int64_t>& d) {
    if (d.empty()) s->ReshapeAsScalar();
    else s->Reshape(d);
}
// numpy multidirectional broadcasting of two shapes, aligned at the last dimension; false when they do not match
static bool BroadcastDims(const std::vector<int64_t>& a, const std::vector<int64_t>& b, std::vector<int64_t>* out) {
    const size_t n = std::max(a.size(), b.size());
    out->assign(n, 1);
    for (size_t i = 0; i < n; ++i) {
        const int64_t da = i < n - a.size() ? 1 : a[i - (n - a.size())];
        const int64_t db = i < n - b.size() ? 1 : b[i - (n - b.size())];
        if (da != db && da != 1 && db != 1) return false;
        (*out)[i] = da == 1 ? db : da;
    }
    return true;
}
// element strides of `src` seen through the broadcast shape `out` (0 where src is broadcast)
static std::vector<int64_t> BroadcastStrides(const std::vector<int64_t>& src, const std::vector<int64_t>& out) {
    std::vector<int64_t> st(out.size(), 0);
    int64_t run = 1;
    for (size_t k = 0; k < src.size(); ++k) {
        const size_t si = src.size() - 1 - k, oi = out.size() - 1 - k;
        st[oi] = src[si] == 1 ? 0 : run;
        run *= src[si];
    }
    return st;
}

// ---------------------------------------------------------------- MatMul
// C[M, N] (+)= A[M, K] * B[K, N], row-major. Register tile of 4 rows x 32 columns, the k loop innermost over whole B
// rows so that every load is contiguous; compiled for AVX-512, AVX2+FMA and baseline x86-64 and picked at load time.
template <int ROWS>
__attribute__((always_inline)) static inline void GemmMicro(const float* __restrict a, const float* __restrict b,
                                                            float* __restrict c, int64_t K, int64_t lda, int64_t ldb,
                                                            int64_t ldc, int cols) {
    constexpr int CT = 32;
    float acc[ROWS][CT];
    for (int r = 0; r < ROWS; ++r)
        for (int j = 0; j < CT; ++j) acc[r][j] = 0.f;
    if (cols == CT) {
        for (int64_t k = 0; k < K; ++k) {
            const float* br = b + k * ldb;
            for (int r = 0; r < ROWS; ++r) {
                const float av = a[r * lda + k];
                for (int j = 0; j < CT; ++j) acc[r][j] += av * br[j];
            }
        }
    } else {
        for (int64_t k = 0; k < K; ++k) {
            const float* br = b + k * ldb;
            for (int r = 0; r < ROWS; ++r) {
                const float av = a[r * lda + k];
                for (int j = 0; j < cols; ++j) acc[r][j] += av * br[j];
            }
        }
    }
    for (int r = 0; r < ROWS; ++r)
        for (int j = 0; j < cols; ++j) c[r * ldc + j] = acc[r][j];
}

__attribute__((target_clones("avx512f", "avx2,fma", "default"))) static void GemmTile(
    const float* __restrict a, const float* __restrict b, float* __restrict c, int64_t m0, int64_t m1, int64_t n0,
    int64_t n1, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
    constexpr int RT = 4, CT = 32;
    for (int64_t i0 = m0; i0 < m1; i0 += RT) {
        const int rows = (int)std::min<int64_t>(RT, m1 - i0);
        for (int64_t j0 = n0; j0 < n1; j0 += CT) {
            const int cols = (int)std::min<int64_t>(CT, n1 - j0);
            const float* at = a + i0 * lda;
            const float* bt = b + j0;
            float* ct = c + i0 * ldc + j0;
            switch (rows) {
                case 4: GemmMicro<4>(at, bt, ct, K, lda, ldb, ldc, cols); break;
                case 3: GemmMicro<3>(at, bt, ct, K, lda, ldb, ldc, cols); break;
                case 2: GemmMicro<2>(at, bt, ct, K, lda, ldb, ldc, cols); break;
                default: GemmMicro<1>(at, bt, ct, K, lda, ldb, ldc, cols); break;
            }
        }
    }
}

class MatMulKernel final : public X86Kernel {
public:
    using X86Kernel::X86Kernel;
    RetCode Reshape(InputOutputInfo* info) const override {
        if (info->GetInputCount() != 2) {
            LOG(DEBUG) << "ERROR: input count[" << info->GetInputCount() << "] != 2.";
            return RC_INVALID_VALUE;
        }
        auto A = info->GetInput<TensorImpl>(0), B = info->GetInput<TensorImpl>(1);
        auto Y = info->GetOutput<TensorImpl>(0);
        if (!A || !B || !Y) return RC_NOT_FOUND;
        std::vector<int64_t> a = DimsOf(*A->GetShape()), b = DimsOf(*B->GetShape());
        if (a.empty() || b.empty()) return RC_INVALID_VALUE;
        const bool a_vec = a.size() == 1, b_vec = b.size() == 1; // numpy: a vector is promoted and the added dim dropped
        if (a_vec) a.insert(a.begin(), 1);
        if (b_vec) b.push_back(1);
        if (a.back() != b[b.size() - 2]) {
            LOG(DEBUG) << "ERROR: cannot broadcast.";
            return RC_INVALID_VALUE;
        }
        std::vector<int64_t> batch;
        if (!BroadcastDims(std::vector<int64_t>(a.begin(), a.end() - 2), std::vector<int64_t>(b.begin(), b.end() - 2), &batch)) {
            LOG(DEBUG) << "ERROR: cannot broadcast.";
            return RC_INVALID_VALUE;
        }
        std::vector<int64_t> out = batch;
        if (!a_vec) out.push_back(a[a.size() - 2]);
        if (!b_vec) out.push_back(b.back());
        SetDims(Y->GetShape(), out);
        Y->GetShape()->SetDataType(A->GetShape()->GetDataType());
        return RC_SUCCESS;
    }

protected:
    RetCode DoExecute(KernelExecContext* ctx) override {
        X86_REQUIRED_INPUT(A, 0);
        X86_REQUIRED_INPUT(B, 1);
        X86_REQUIRED_OUTPUT(Y, 0);
        auto rc = ReallocOnHost(Y);
        if (rc != RC_SUCCESS) return rc;
        if (!IsFp32Ndarray(A) || !IsFp32Ndarray(B)) {
            LOG(ERROR) << "only support fp32 ndarray now.";
            return RC_UNSUPPORTED;
        }
        std::vector<int64_t> a = DimsOf(*A->GetShape()), b = DimsOf(*B->GetShape());
        if (a.size() == 1) a.insert(a.begin(), 1);
        if (b.size() == 1) b.push_back(1);
        const int64_t M = a[a.size() - 2], K = a.back(), N = b.back();
        const std::vector<int64_t> ab(a.begin(), a.end() - 2), bb(b.begin(), b.end() - 2);
        std::vector<int64_t> batch;
        BroadcastDims(ab, bb, &batch);
        const std::vector<int64_t> sa = BroadcastStrides(ab, batch), sb = BroadcastStrides(bb, batch);
        int64_t nb = 1;
        for (auto d : batch) nb *= d;
        const float* pa = A->GetBufferPtr<float>();
        const float* pb = B->GetBufferPtr<float>();
        float* py = Y->GetBufferPtr<float>();
        if (nb == 0 || M == 0 || N == 0) return RC_SUCCESS;
        // work items: (batch entry, row block, column block), sized so that every thread gets several
        const int64_t mb = 32, nbk = 256;
        const int64_t mblocks = (M + mb - 1) / mb, nblocks = (N + nbk - 1) / nbk;
        const int64_t items = nb * mblocks * nblocks;
#pragma omp parallel for schedule(static)
        for (int64_t it = 0; it < items; ++it) {
            const int64_t bi = it / (mblocks * nblocks), rem = it % (mblocks * nblocks);
            const int64_t mi = rem / nblocks, ni = rem % nblocks;
            int64_t oa = 0, ob = 0, x = bi;
            for (int d = (int)batch.size() - 1; d >= 0; --d) {
                const int64_t i = x % batch[d];
                x /= batch[d];
                oa += i * sa[d];
                ob += i * sb[d];
            }
            GemmTile(pa + oa * M * K, pb + ob * K * N, py + bi * M * N, mi * mb, std::min(M, (mi + 1) * mb), ni * nbk,
                     std::min(N, (ni + 1) * nbk), K, K, N, N);
        }
        return RC_SUCCESS;
    }
};

// ---------------------------------------------------------------- Add / Mul
enum ArithOp { ARITH_ADD, ARITH_MUL };

template <ArithOp OP>
class ArithmeticKernel final : public X86Kernel {
public:
    using X86Kernel::X86Kernel;
    RetCode Reshape(InputOutputInfo* info) const override {
        auto A = info->GetInput<TensorImpl>(0), B = info->GetInput<TensorImpl>(1);
        auto C = info->GetOutput<TensorImpl>(0);
        if (!A || !B || !C) return RC_NOT_FOUND;
        std::vector<int64_t> out;
        if (!BroadcastDims(DimsOf(*A->GetShape()), DimsOf(*B->GetShape()), &out)) {
            LOG(DEBUG) << "ERROR: cannot broadcast.";
            return RC_INVALID_VALUE;
        }
        SetDims(C->GetShape(), out);
        C->GetShape()->SetDataType(A->GetShape()->GetDataType());
        return RC_SUCCESS;
    }

protected:
    RetCode DoExecute(KernelExecContext* ctx) override {
        X86_REQUIRED_INPUT(A, 0);
        X86_REQUIRED_INPUT(B, 1);
        X86_REQUIRED_OUTPUT(C, 0);
        const std::vector<int64_t> da = DimsOf(*A->GetShape()), db = DimsOf(*B->GetShape()), dc = DimsOf(*C->GetShape());
        // the output takes over an input's buffer when that input dies here and has the output's shape
        // (add_kernel.cc:49-58)
        TensorImpl *lA = A, *lB = B;
        if (ctx->IsLastConsumerOfInput(0) && da == dc && A->GetBufferInfo().IsBufferOwner()) {
            C->TransferBufferFrom(A);
            lA = C;
        } else if (ctx->IsLastConsumerOfInput(1) && db == dc && B->GetBufferInfo().IsBufferOwner()) {
            C->TransferBufferFrom(B);
            lB = C;
        } else {
            auto rc = ReallocOnHost(C);
            if (rc != RC_SUCCESS) return rc;
        }
        if (A->GetShape()->GetDataType() != DATATYPE_FLOAT32 || B->GetShape()->GetDataType() != DATATYPE_FLOAT32) {
            LOG(ERROR) << "unsupported datatype: " << GetDataTypeStr(A->GetShape()->GetDataType());
            return RC_UNSUPPORTED;
        }
        const float* pa = lA->GetBufferPtr<float>();
        const float* pb = lB->GetBufferPtr<float>();
        float* pc = C->GetBufferPtr<float>();
        int64_t total = 1;
        for (auto d : dc) total *= d;
        if (total == 0) return RC_SUCCESS;
        const std::vector<int64_t> sa = BroadcastStrides(da, dc), sb = BroadcastStrides(db, dc);
        // rows of the innermost dimension; each operand's row is contiguous (stride 1) or one value (stride 0)
        const int64_t inner = dc.empty() ? 1 : dc.back();
        const int64_t ia = dc.empty() ? 0 : sa.back(), ib = dc.empty() ? 0 : sb.back();
        const int64_t rows = total / inner;
        const int nd = (int)dc.size();
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; ++r) {
            int64_t oa = 0, ob = 0, x = r;
            for (int d = nd - 2; d >= 0; --d) {
                const int64_t i = x % dc[d];
                x /= dc[d];
                oa += i * sa[d];
                ob += i * sb[d];
            }
            const float* ra = pa + oa;
            const float* rb = pb + ob;
            float* rc = pc + r * inner;
            for (int64_t j = 0; j < inner; ++j) {
                const float x0 = ra[j * ia], x1 = rb[j * ib];
                rc[j] = OP == ARITH_ADD ? x0 + x1 : x0 * x1;
            }
        }
        return RC_SUCCESS;
    }
};

// ---------------------------------------------------------------- Softmax
class SoftmaxKernel final : public X86Kernel {
public:
    SoftmaxKernel(const ir::Node* node, const onnx::SoftmaxParam* p) : X86Kernel(node), param_(p) {}
    RetCode Reshape(InputOutputInfo* info) const override {
        auto in = info->GetInput<TensorImpl>(0);
        auto out = info->GetOutput<TensorImpl>(0);
        if (!in || !out) return RC_NOT_FOUND;
        const int64_t nd = in->GetShape()->GetRealDimCount();
        if (param_->axis < -nd || param_->axis >= std::max<int64_t>(nd, 1)) {
            LOG(DEBUG) << "ERROR: axis[" << param_->axis << "] is out of range[" << -nd << ", " << nd << ").";
            return RC_INVALID_VALUE;
        }
        SetDims(out->GetShape(), DimsOf(*in->GetShape()));
        out->GetShape()->SetDataType(in->GetShape()->GetDataType());
        return RC_SUCCESS;
    }

protected:
    RetCode DoExecute(KernelExecContext* ctx) override {
        X86_REQUIRED_INPUT(input, 0);
        X86_REQUIRED_OUTPUT(output, 0);
        auto rc = ReallocOnHost(output);
        if (rc != RC_SUCCESS) return rc;
        if (input->GetShape()->GetDataType() != DATATYPE_FLOAT32) {
            LOG(ERROR) << "unsupported data type " << GetDataTypeStr(input->GetShape()->GetDataType()) << ".";
            return RC_UNSUPPORTED;
        }
        const std::vector<int64_t> d = DimsOf(*input->GetShape());
        const int nd = (int)d.size();
        const int axis = nd == 0 ? 0 : (param_->axis < 0 ? param_->axis + nd : param_->axis);
        int64_t outer = 1, len = 1, inner = 1;
        for (int i = 0; i < axis; ++i) outer *= d[i];
        if (GetNode()->GetType().version < 13) { // the input is coerced to [prod(d[:axis]), prod(d[axis:])]
            for (int i = axis; i < nd; ++i) len *= d[i];
        } else { // along `axis` only
            len = nd ? d[axis] : 1;
            for (int i = axis + 1; i < nd; ++i) inner *= d[i];
        }
        const float* src = input->GetBufferPtr<float>();
        float* dst = output->GetBufferPtr<float>();
        if (outer * len * inner == 0) return RC_SUCCESS;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < outer * inner; ++r) {
            const int64_t o = r / inner, in = r % inner;
            const float* s = src + o * len * inner + in;
            float* t = dst + o * len * inner + in;
            float mx = -INFINITY;
            for (int64_t j = 0; j < len; ++j) mx = std::max(mx, s[j * inner]);
            float sum = 0.f;
            for (int64_t j = 0; j < len; ++j) {
                const float e = expf(s[j * inner] - mx);
                t[j * inner] = e;
                sum += e;
            }
            const float inv = 1.0f / sum;
            for (int64_t j = 0; j < len; ++j) t[j * inner] *= inv;
        }
        return RC_SUCCESS;
    }

private:
    const onnx::SoftmaxParam* param_;
};

// ---------------------------------------------------------------- Transpose
class TransposeKernel final : public X86Kernel {
public:
    TransposeKernel(const ir::Node* node, const onnx::TransposeParam* p) : X86Kernel(node), param_(p) {}
    RetCode Reshape(InputOutputInfo* info) const override {
        auto in = info->GetInput<TensorImpl>(0);
        auto out = info->GetOutput<TensorImpl>(0);
        if (!in || !out) return RC_NOT_FOUND;
        const std::vector<int64_t> d = DimsOf(*in->GetShape());
        std::vector<int32_t> perm;
        if (!Perm((int)d.size(), &perm)) {
            LOG(DEBUG) << "ERROR: perm does not match the input's " << d.size() << " dimensions.";
            return RC_INVALID_VALUE;
        }
        std::vector<int64_t> od(d.size());
        for (size_t i = 0; i < d.size(); ++i) od[i] = d[perm[i]];
        SetDims(out->GetShape(), od);
        out->GetShape()->SetDataType(in->GetShape()->GetDataType());
        return RC_SUCCESS;
    }

protected:
    RetCode DoExecute(KernelExecContext* ctx) override {
        X86_REQUIRED_INPUT(data, 0);
        X86_REQUIRED_OUTPUT(transposed, 0);
        auto rc = ReallocOnHost(transposed);
        if (rc != RC_SUCCESS) return rc;
        if (GetSizeOfDataType(data->GetShape()->GetDataType()) != 4) {
            LOG(ERROR) << "unsupported data type " << GetDataTypeStr(data->GetShape()->GetDataType()) << ".";
            return RC_UNSUPPORTED;
        }
        const std::vector<int64_t> d = DimsOf(*data->GetShape()), od = DimsOf(*transposed->GetShape());
        std::vector<int32_t> perm;
        Perm((int)d.size(), &perm);
        const int nd = (int)d.size();
        std::vector<int64_t> in_stride(nd, 1), st(nd, 1);
        for (int i = nd - 2; i >= 0; --i) in_stride[i] = in_stride[i + 1] * d[i + 1];
        for (int i = 0; i < nd; ++i) st[i] = in_stride[perm[i]]; // input stride of output dimension i
        int64_t total = 1;
        for (auto x : od) total *= x;
        if (total == 0) return RC_SUCCESS;
        const uint32_t* src = data->GetBufferPtr<uint32_t>();
        uint32_t* dst = transposed->GetBufferPtr<uint32_t>();
        const int64_t inner = nd ? od.back() : 1, is = nd ? st.back() : 0, rows = total / inner;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; ++r) {
            int64_t off = 0, x = r;
            for (int i = nd - 2; i >= 0; --i) {
                off += (x % od[i]) * st[i];
                x /= od[i];
            }
            for (int64_t j = 0; j < inner; ++j) dst[r * inner + j] = src[off + j * is];
        }
        return RC_SUCCESS;
    }

private:
    bool Perm(int nd, std::vector<int32_t>* perm) const { // empty = reversed dimensions (reshape_transpose.cc:29-36)
        *perm = param_->perm;
        if (perm->empty())
            for (int i = 0; i < nd; ++i) perm->push_back(nd - 1 - i);
        if ((int)perm->size() != nd) return false;
        std::vector<bool> seen(nd, false);
        for (auto& p : *perm) {
            if (p < 0) p += nd;
            if (p < 0 || p >= nd || seen[p]) return false;
            seen[p] = true;
        }
        return true;
    }
    const onnx::TransposeParam* param_;
};

// ---------------------------------------------------------------- ops
class X86OptKernel : public OptKernel {
public:
    X86OptKernel(const ir::Node* node) : OptKernel(node) {}
    virtual RetCode Init(const ir::Graph* graph) = 0;

protected:
    template <typename T>
    RetCode GenericLoadParam(const ir::Graph* graph, std::shared_ptr<T>* param) {
        auto it = graph->data->attrs.find(GetNode()->GetId());
        if (it == graph->data->attrs.end()) {
            LOG(ERROR) << "cannot find attr for op[" << GetNode()->GetName() << "]";
            return RC_NOT_FOUND;
        }
        *param = std::static_pointer_cast<T>(it->second);
        return RC_SUCCESS;
    }
};

template <typename K>
class ParamlessOp final : public X86OptKernel {
public:
    using X86OptKernel::X86OptKernel;
    RetCode Init(const ir::Graph*) override { return RC_SUCCESS; }
    KernelImpl* CreateKernelImpl() const override { return new K(GetNode()); }
};
class SoftmaxOp final : public X86OptKernel {
public:
    using X86OptKernel::X86OptKernel;
    RetCode Init(const ir::Graph* graph) override { return GenericLoadParam(graph, &param_); }
    KernelImpl* CreateKernelImpl() const override { return new SoftmaxKernel(GetNode(), param_.get()); }

private:
    std::shared_ptr<onnx::SoftmaxParam> param_;
};
class TransposeOp final : public X86OptKernel {
public:
    using X86OptKernel::X86OptKernel;
    RetCode Init(const ir::Graph* graph) override { return GenericLoadParam(graph, &param_); }
    KernelImpl* CreateKernelImpl() const override { return new TransposeKernel(GetNode(), param_.get()); }

private:
    std::shared_ptr<onnx::TransposeParam> param_;
};

typedef X86OptKernel* (*OptKernelCreator)(const ir::Node*);
static utils::OpInfoManager<OptKernelCreator>& OptKernelCreatorManager() {
    static utils::OpInfoManager<OptKernelCreator> mgr;
    return mgr;
}
template <typename T>
static X86OptKernel* GenericCreateOptKernel(const ir::Node* node) {
    return new T(node);
}
template <typename T>
static void RegisterOptKernelCreator(const std::string& domain, const std::string& type, uint64_t first, uint64_t last) {
    if (last < first) { // x86_ops.cc: an invalid range is a programming error
        LOG(ERROR) << "register op[" << domain << ":" << type << "] failed: last version[" << last
                   << "] < first version[" << first << "]";
        exit(-1);
    }
    OptKernelCreatorManager().Register(domain, type, utils::VersionRange{first, last}, GenericCreateOptKernel<T>);
}
static void RegisterBuiltinOpImpls() { // x86_ops.cc:146,194,199,232,246
    static std::once_flag once;
    std::call_once(once, [] {
        RegisterOptKernelCreator<ParamlessOp<ArithmeticKernel<ARITH_ADD>>>("", "Add", 7, 16);
        RegisterOptKernelCreator<ParamlessOp<MatMulKernel>>("", "MatMul", 1, 16);
        RegisterOptKernelCreator<ParamlessOp<ArithmeticKernel<ARITH_MUL>>>("", "Mul", 7, 16);
        RegisterOptKernelCreator<SoftmaxOp>("", "Softmax", 1, 16);
        RegisterOptKernelCreator<TransposeOp>("", "Transpose", 1, 16);
    });
}

// ---------------------------------------------------------------- engine
class X86Engine final : public EngineImpl {
public:
    X86Engine() : EngineImpl("x86") {}
    RetCode Init(const EngineOptions& options) {
        if (options.mm_policy != MM_COMPACT && options.mm_policy != MM_MRU && options.mm_policy != MM_PLAIN) {
            LOG(ERROR) << "unknown mm_policy " << options.mm_policy;
            return RC_INVALID_VALUE;
        }
        return RC_SUCCESS;
    }
    EngineContext* CreateEngineContext() override { return new X86EngineContext(); }
    bool Supports(const ir::Node* node) const override {
        auto& type = node->GetType();
        return OptKernelCreatorManager().Find(type.domain, type.name, type.version) != nullptr;
    }
    RetCode ProcessGraph(ir::Graph* graph, RuntimePartitionInfo* info) override {
        for (auto& node : graph->topo->nodes) {
            auto& type = node.GetType();
            auto creator = OptKernelCreatorManager().Find(type.domain, type.name, type.version);
            if (!creator) {
                LOG(ERROR) << "cannot find creator for node[" << node.GetName() << "] of type[" << type.domain << ":"
                           << type.name << ":" << type.version << "]";
                return RC_NOT_FOUND;
            }
            std::unique_ptr<X86OptKernel> op((*creator)(&node));
            auto rc = op->Init(graph);
            if (rc != RC_SUCCESS) {
                LOG(ERROR) << "Init for kernel[" << node.GetName() << "] failed: " << GetRetCodeStr(rc);
                return rc;
            }
            info->kernels[node.GetId()] = std::move(op);
        }
        return RC_SUCCESS;
    }
    RetCode Configure(uint32_t option, ...) override {
        va_list args;
        va_start(args, option);
        RetCode rc = RC_SUCCESS;
        switch (option) {
            case ENGINE_CONF_GRAPH_FUSION: config_.enable_graph_fusion = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_TENSOR_DEBUG: config_.enable_tensor_debug = va_arg(args, uint32_t) ? true : false; break;
            case ENGINE_CONF_DEBUG_DATA_DIR: config_.debug_data_dir = va_arg(args, const char*); break;
            default:
                LOG(ERROR) << "invalid option[" << option << "] >= [" << (uint32_t)ENGINE_CONF_MAX << "]";
                rc = RC_INVALID_VALUE;
        }
        va_end(args);
        return rc;
    }

private:
    EngineConfig config_;
};

Engine* EngineFactory::Create(const EngineOptions& options) {
    RegisterBuiltinOpImpls();
    auto engine = new X86Engine();
    if (engine->Init(options) != RC_SUCCESS) {
        delete engine;
        return nullptr;
    }
    return engine;
}

void SetGlobalOmpNumThreads(int n) {
    if (n > 0) omp_set_num_threads(n);
}

int GetGlobalOmpNumThreads() {
    return omp_get_max_threads();
}

}}} // namespace ppl::nn::x86
