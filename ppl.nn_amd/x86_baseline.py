"""Host-side driver of the x86 engine: the fp32 ONNX attention subgraph (Transpose, MatMul, Mul, Add, Softmax, MatMul)
loaded through the engine library's ONNX reader and run on the host cores, the way `pplnn --use-x86 --onnx-model ...
--num-threads N` runs a model in the reference (tools/pplnn.cc:332,377-380). It is the CPU baseline the GPU path is
reported next to, labelled "PPLNN-x86-semantics baseline (own kernels)": the reference's x86 arithmetic lives in its
un-vendored ppl.kernel.cpu."""
import ctypes as C

import numpy as np

from . import load_engine_library, onnx_writer


class X86Session:
    """One runtime of the x86 engine over a serialized ONNX model."""

    def __init__(self, model_bytes, num_threads=0):
        self.eng = eng = load_engine_library()
        if num_threads:
            eng.pplnn_x86_set_num_threads(int(num_threads))
        self.engine = eng.pplnn_x86_engine_create()
        if not self.engine:
            raise RuntimeError("x86 engine: create failed")
        self.builder = eng.pplnn_hip_builder_create()
        self._check(eng.pplnn_hip_builder_load_model(self.builder, model_bytes, len(model_bytes)), "load model")
        self._check(eng.pplnn_hip_builder_set_engine(self.builder, self.engine), "set resources")
        self._check(eng.pplnn_hip_builder_preprocess(self.builder), "preprocess")
        self.rt = eng.pplnn_hip_builder_create_runtime(self.builder)
        if not self.rt:
            raise RuntimeError("x86 engine: create runtime failed: " + eng.pplnn_hip_last_error().decode())
        self._keep = []

    def _check(self, rc, what):
        if rc:
            raise RuntimeError(f"x86 engine: {what} failed (rc {rc}): {self.eng.pplnn_hip_last_error().decode()}")

    @property
    def num_threads(self):
        return self.eng.pplnn_x86_get_num_threads()

    def set_input(self, i, a):
        """Borrows `a` (C-contiguous float32) as input i: no copy, like Tensor::SetBufferPtr."""
        assert a.dtype == np.float32 and a.flags.c_contiguous
        t = self.eng.pplnn_hip_runtime_input(self.rt, i)
        dims = (C.c_int64 * a.ndim)(*a.shape)
        self.eng.pplnn_hip_tensor_reshape(t, dims, a.ndim)
        self.eng.pplnn_hip_tensor_set_buffer_ptr(t, a.ctypes.data)
        self._keep.append(a)

    def run(self):
        self._check(self.eng.pplnn_hip_runtime_run(self.rt), "run")
        self._keep = self._keep[-8:]

    def output(self, i=0):
        t = self.eng.pplnn_hip_runtime_output(self.rt, i)
        dims = (C.c_int64 * 8)()
        n = self.eng.pplnn_hip_tensor_dims(t, dims, 8)
        out = np.empty(tuple(dims[:n]), np.float32)
        self._check(self.eng.pplnn_hip_tensor_copy_to_host(t, out.ctypes.data), "copy output")
        return out

    def close(self):
        self.eng.pplnn_hip_runtime_destroy(self.rt)
        self.eng.pplnn_hip_builder_destroy(self.builder)
        self.eng.pplnn_hip_engine_destroy(self.engine)
        self.rt = self.builder = self.engine = None


def causal_mask(lq, lk):
    """Additive fp32 mask [lq, lk]: query i (the last lq of lk positions) sees keys j <= (lk - lq) + i, -inf elsewhere."""
    i = np.arange(lq)[:, None]
    j = np.arange(lk)[None, :]
    return np.where(j <= (lk - lq) + i, 0.0, -np.inf).astype(np.float32)


class AttentionBaseline:
    """softmax(Q K^T / sqrt(d) + mask) V per sequence through the x86 engine. q [H, Lq, d]; k, v [KVH, Lk, d] float32."""

    def __init__(self, head_dim, num_threads=0):
        self.head_dim = head_dim
        self.mha = X86Session(onnx_writer.attention_fp32_model(head_dim, rank=3), num_threads)
        self.gqa = X86Session(onnx_writer.attention_fp32_model(head_dim, rank=4), num_threads)

    @property
    def num_threads(self):
        return self.mha.num_threads

    def run(self, q, k, v, mask):
        H, KVH = q.shape[0], k.shape[0]
        if H == KVH:
            s = self.mha
            ins = (q, k, v, mask)
        else:  # grouped heads: MatMul's batch broadcasting shares each kv head among its query heads
            s = self.gqa
            rep = H // KVH
            ins = (q.reshape(KVH, rep, *q.shape[1:]), k.reshape(KVH, 1, *k.shape[1:]), v.reshape(KVH, 1, *v.shape[1:]),
                   mask)
        for i, a in enumerate(ins):
            s.set_input(i, np.ascontiguousarray(a, dtype=np.float32))
        s.run()
        return s.output(0).reshape(q.shape)

    def close(self):
        self.mha.close()
        self.gqa.close()
