"""Torch-level convenience layer over the 3+1-stage C API.

Each `*Plan` object is one operator descriptor: it is created from example
tensors (stage 2, where the library validates shapes, strides and dtypes),
can be launched any number of times on tensors of that layout (stage 4) and
destroys the descriptor when closed.  `Context` owns a handle (stage 1).

Launches go to the stream given (a raw hipStream_t value, e.g.
`torch.cuda.current_stream().cuda_stream`); None is the null stream, which is
what the reference's harness passes.  Nothing here synchronises.
"""
import ctypes

from .devices import DeviceEnum
from .liboperators import (
    infiniopAddDescriptor_t,
    infiniopCausalSoftmaxDescriptor_t,
    infiniopRearrangeDescriptor_t,
    infiniopAddRMSNormDescriptor_t,
    infiniopAttentionDescriptor_t,
    infiniopMatmulDescriptor_t,
    infiniopMLPDescriptor_t,
    infiniopRMSNormDescriptor_t,
    infiniopRandomSampleDescriptor_t,
    infiniopRoPEDescriptor_t,
    infiniopSwiGLUDescriptor_t,
    open_lib,
)
from .utils import check_error, create_handle, destroy_handle, destroy_tensor, to_tensor


class _Plan:
    _destroy = None

    def __init__(self, ctx):
        self.ctx = ctx
        self.lib = ctx.lib
        self.desc = None

    def _describe(self, *tensors):
        cts = [to_tensor(t, self.lib) for t in tensors]
        return cts

    def _release(self, cts):
        for ct in cts:
            destroy_tensor(self.lib, ct)

    def close(self):
        if self.desc is not None:
            check_error(getattr(self.lib, self._destroy)(self.desc))
            self.desc = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


class AddPlan(_Plan):
    _destroy = "infiniopDestroyAddDescriptor"

    def __init__(self, ctx, c, a, b):
        super().__init__(ctx)
        cts = self._describe(c, a, b)
        desc = infiniopAddDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateAddDescriptor(ctx.handle, ctypes.byref(desc), *[ct.descriptor for ct in cts]))
        finally:
            self._release(cts)
        self.desc = desc

    def __call__(self, c, a, b, stream=None):
        check_error(self.lib.infiniopAdd(self.desc, c.data_ptr(), a.data_ptr(), b.data_ptr(), stream))
        return c


class SwiGLUPlan(_Plan):
    _destroy = "infiniopDestroySwiGLUDescriptor"

    def __init__(self, ctx, c, a, b):
        super().__init__(ctx)
        cts = self._describe(c, a, b)
        desc = infiniopSwiGLUDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateSwiGLUDescriptor(ctx.handle, ctypes.byref(desc), *[ct.descriptor for ct in cts]))
        finally:
            self._release(cts)
        self.desc = desc

    def __call__(self, c, a, b, stream=None):
        check_error(self.lib.infiniopSwiGLU(self.desc, c.data_ptr(), a.data_ptr(), b.data_ptr(), stream))
        return c


class RMSNormPlan(_Plan):
    _destroy = "infiniopDestroyRMSNormDescriptor"

    def __init__(self, ctx, y, x, w, epsilon):
        super().__init__(ctx)
        cts = self._describe(y, x, w)
        desc = infiniopRMSNormDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateRMSNormDescriptor(ctx.handle, ctypes.byref(desc), *[ct.descriptor for ct in cts], epsilon))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetRMSNormWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value  # 0 for this library; the query is part of the calling sequence

    def __call__(self, y, x, w, stream=None):
        check_error(self.lib.infiniopRMSNorm(self.desc, None, self.workspace_size, y.data_ptr(), x.data_ptr(), w.data_ptr(), stream))
        return y


class AddRMSNormPlan(_Plan):
    """c = a + b; y = RMSNorm(c) * w in one pass (the reference issues Add, then RMSNorm)."""

    _destroy = "infiniopDestroyAddRMSNormDescriptor"

    def __init__(self, ctx, y, c, a, b, w, epsilon):
        super().__init__(ctx)
        cts = self._describe(y, c, a, b, w)
        desc = infiniopAddRMSNormDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateAddRMSNormDescriptor(ctx.handle, ctypes.byref(desc), *[ct.descriptor for ct in cts], epsilon))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetAddRMSNormWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value

    def __call__(self, y, c, a, b, w, stream=None):
        check_error(self.lib.infiniopAddRMSNorm(self.desc, None, self.workspace_size, y.data_ptr(), c.data_ptr(), a.data_ptr(), b.data_ptr(), w.data_ptr(), stream))
        return y, c


class MatmulPlan(_Plan):
    """c = alpha * a @ b + beta * c (2-D or batched 3-D, row- or column-major operands)."""

    _destroy = "infiniopDestroyMatmulDescriptor"

    def __init__(self, ctx, c, a, b, alpha=1.0, beta=0.0):
        super().__init__(ctx)
        cts = self._describe(c, a, b)
        desc = infiniopMatmulDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateMatmulDescriptor(ctx.handle, ctypes.byref(desc), cts[0].descriptor, alpha,
                                                                cts[1].descriptor, cts[2].descriptor, beta))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetMatmulWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value
        # 0 but for few columns summed over very many k (the weighted values of a decoding attention)
        self.workspace = None
        if self.workspace_size:
            import torch

            self.workspace = torch.empty(self.workspace_size, dtype=torch.uint8, device=c.device)

    def __call__(self, c, a, b, stream=None, use_workspace=True):
        ws = self.workspace.data_ptr() if (self.workspace is not None and use_workspace) else None
        check_error(self.lib.infiniopMatmul(self.desc, ws, self.workspace_size if ws else 0, c.data_ptr(), a.data_ptr(), b.data_ptr(), stream))
        return c


class MLPPlan(_Plan):
    """y = alpha * SwiGLU(x @ w12) @ w3 (+ y); owns the workspace the composite asks for."""

    _destroy = "infiniopDestroyMLPDescriptor"

    def __init__(self, ctx, y, x, w12, w3, alpha=1.0, residual=False):
        import torch

        super().__init__(ctx)
        cts = self._describe(y, x, w12, w3)
        desc = infiniopMLPDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateMLPDescriptor(ctx.handle, ctypes.byref(desc), *[ct.descriptor for ct in cts], alpha,
                                                             ctypes.c_char(b"\x01" if residual else b"\x00")))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetMLPWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value
        self.workspace = torch.empty(max(1, size.value), dtype=torch.uint8, device=x.device)

    def __call__(self, y, x, w12, w3, stream=None):
        check_error(self.lib.infiniopMLP(self.desc, self.workspace.data_ptr(), self.workspace_size, y.data_ptr(), x.data_ptr(),
                                         w12.data_ptr(), w3.data_ptr(), stream))
        return y


class AttentionPlan(_Plan):
    """k, v -> caches at `pos`; out = softmax_causal(q K^T / sqrt(d)) V; owns the workspace."""

    _destroy = "infiniopDestroyAttentionDescriptor"

    def __init__(self, ctx, out, q, k, v, k_cache, v_cache, pos):
        import torch

        super().__init__(ctx)
        cts = self._describe(out, q, k, v, k_cache, v_cache)
        desc = infiniopAttentionDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateAttentionDescriptor(ctx.handle, ctypes.byref(desc), *[ct.descriptor for ct in cts], pos))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetAttentionWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value
        self.workspace = torch.empty(max(1, size.value), dtype=torch.uint8, device=q.device)

    def __call__(self, out, q, k, v, k_cache, v_cache, stream=None):
        check_error(self.lib.infiniopAttention(self.desc, self.workspace.data_ptr(), self.workspace_size, out.data_ptr(), q.data_ptr(),
                                               k.data_ptr(), v.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), stream))
        return out


class RoPEPlan(_Plan):
    _destroy = "infiniopDestroyRoPEDescriptor"

    def __init__(self, ctx, t, pos_ids, sin_table, cos_table):
        super().__init__(ctx)
        cts = self._describe(t, pos_ids, sin_table, cos_table)
        desc = infiniopRoPEDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateRoPEDescriptor(ctx.handle, ctypes.byref(desc), *[ct.descriptor for ct in cts]))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetRoPEWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value

    def __call__(self, t, pos_ids, sin_table, cos_table, stream=None):
        check_error(self.lib.infiniopRoPE(self.desc, None, self.workspace_size, t.data_ptr(), pos_ids.data_ptr(),
                                          sin_table.data_ptr(), cos_table.data_ptr(), stream))
        return t


class CausalSoftmaxPlan(_Plan):
    _destroy = "infiniopDestroyCausalSoftmaxDescriptor"

    def __init__(self, ctx, y):
        super().__init__(ctx)
        cts = self._describe(y)
        desc = infiniopCausalSoftmaxDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateCausalSoftmaxDescriptor(ctx.handle, ctypes.byref(desc), cts[0].descriptor))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetCausalSoftmaxWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value
        # 0 for every shape but few long rows (decoding over a long context), whose parts meet in the workspace
        self.workspace = None
        if self.workspace_size:
            import torch

            self.workspace = torch.empty(self.workspace_size, dtype=torch.uint8, device=y.device)

    def __call__(self, y, stream=None, use_workspace=True):
        ws = self.workspace.data_ptr() if (self.workspace is not None and use_workspace) else None
        check_error(self.lib.infiniopCausalSoftmax(self.desc, ws, self.workspace_size if ws else 0, y.data_ptr(), stream))
        return y


class RandomSamplePlan(_Plan):
    """One token index drawn from a 1-D fp16 logits tensor into a uint64 (or
    int64, whose bits are the same) result tensor.  Owns the workspace the
    library asks for; with use_workspace=False none is passed and the library
    serves the call with one workgroup."""
    _destroy = "infiniopDestroyRandomSampleDescriptor"

    def __init__(self, ctx, result, probs, use_workspace=True):
        import torch

        super().__init__(ctx)
        cts = self._describe(result, probs)
        desc = infiniopRandomSampleDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateRandomSampleDescriptor(ctx.handle, ctypes.byref(desc), cts[0].descriptor, cts[1].descriptor))
        finally:
            self._release(cts)
        self.desc = desc
        size = ctypes.c_uint64(0)
        check_error(self.lib.infiniopGetRandomSampleWorkspaceSize(desc, ctypes.byref(size)))
        self.workspace_size = size.value if use_workspace else 0
        self.workspace = torch.empty(self.workspace_size, dtype=torch.uint8, device=probs.device) if self.workspace_size else None

    def __call__(self, result, probs, random_val, topp, topk, temperature, stream=None):
        check_error(self.lib.infiniopRandomSample(self.desc, self.workspace.data_ptr() if self.workspace is not None else None,
                                                  self.workspace_size, result.data_ptr(), probs.data_ptr(),
                                                  random_val, topp, topk, temperature, stream))
        return result

    def no_alloc(self, result, probs, random_val, topp, topk, temperature, stream=None):
        """The same draw through the entry point that neither takes a workspace
        nor allocates: the library's own array on the GPU carries the lists."""
        check_error(self.lib.infiniopRandomSampleNoAlloc(self.desc, result.data_ptr(), probs.data_ptr(),
                                                         random_val, topp, topk, temperature, stream))
        return result


class RearrangePlan(_Plan):
    _destroy = "infiniopDestroyRearrangeDescriptor"

    def __init__(self, ctx, dst, src):
        super().__init__(ctx)
        cts = self._describe(dst, src)
        desc = infiniopRearrangeDescriptor_t()
        try:
            check_error(self.lib.infiniopCreateRearrangeDescriptor(ctx.handle, ctypes.byref(desc), cts[0].descriptor, cts[1].descriptor))
        finally:
            self._release(cts)
        self.desc = desc

    def __call__(self, dst, src, stream=None):
        check_error(self.lib.infiniopRearrange(self.desc, dst.data_ptr(), src.data_ptr(), stream))
        return dst


class Context:
    """A library handle on one GPU plus one-shot forms of the four operators."""

    def __init__(self, device_id=0, lib=None, device=DeviceEnum.DEVICE_AMD):
        self.lib = lib or open_lib()
        self.handle = create_handle(self.lib, device, device_id)

    def close(self):
        if self.handle is not None:
            destroy_handle(self.lib, self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def add(self, c, a, b, stream=None):
        with AddPlan(self, c, a, b) as plan:
            return plan(c, a, b, stream)

    def swiglu(self, c, a, b, stream=None):
        with SwiGLUPlan(self, c, a, b) as plan:
            return plan(c, a, b, stream)

    def rms_norm(self, y, x, w, epsilon=1e-5, stream=None):
        with RMSNormPlan(self, y, x, w, epsilon) as plan:
            return plan(y, x, w, stream)

    def add_rms_norm(self, y, c, a, b, w, epsilon=1e-5, stream=None):
        with AddRMSNormPlan(self, y, c, a, b, w, epsilon) as plan:
            return plan(y, c, a, b, w, stream)

    def matmul(self, c, a, b, alpha=1.0, beta=0.0, stream=None):
        with MatmulPlan(self, c, a, b, alpha, beta) as plan:
            return plan(c, a, b, stream)

    def mlp(self, y, x, w12, w3, alpha=1.0, residual=False, stream=None):
        import torch

        with MLPPlan(self, y, x, w12, w3, alpha, residual) as plan:
            out = plan(y, x, w12, w3, stream)
            torch.cuda.synchronize()  # the plan's workspace must outlive the work queued on it
            return out

    def attention(self, out, q, k, v, k_cache, v_cache, pos, stream=None):
        import torch

        with AttentionPlan(self, out, q, k, v, k_cache, v_cache, pos) as plan:
            res = plan(out, q, k, v, k_cache, v_cache, stream)
            torch.cuda.synchronize()  # the plan's workspace must outlive the work queued on it
            return res

    def rearrange(self, dst, src, stream=None):
        with RearrangePlan(self, dst, src) as plan:
            return plan(dst, src, stream)

    def random_sample(self, result, probs, random_val, topp, topk, temperature, stream=None, use_workspace=True):
        import torch

        with RandomSamplePlan(self, result, probs, use_workspace) as plan:
            res = plan(result, probs, random_val, topp, topk, temperature, stream)
            torch.cuda.synchronize()  # the plan's workspace must outlive the work queued on it
            return res

    def causal_softmax(self, y, stream=None, use_workspace=True):
        with CausalSoftmaxPlan(self, y) as plan:
            return plan(y, stream, use_workspace)

    def rope(self, t, pos_ids, sin_table, cos_table, stream=None):
        with RoPEPlan(self, t, pos_ids, sin_table, cos_table) as plan:
            return plan(t, pos_ids, sin_table, cos_table, stream)


def sin_cos_table(rows, head_dim, theta, device="cpu"):
    """fp32 sin/cos tables [rows, head_dim] with each frequency repeated for
    the two members of a pair, all arithmetic in fp32 (the table layout the
    reference's harness builds, operatorspy/tests/rotary_embedding.py:54-64)."""
    import torch

    pos = torch.arange(0, rows, dtype=torch.float32, device=device)
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device)[: head_dim // 2].float() / head_dim))
    freqs = torch.repeat_interleave(freqs, repeats=2)
    angles = torch.outer(pos, freqs)
    return torch.sin(angles).contiguous(), torch.cos(angles).contiguous()
