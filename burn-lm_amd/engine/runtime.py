"""What parts need from the machine: device, activation dtype, and the matrix product.

Matrix products ``x[M,K] @ w[N,K]^T``:
* float32 weights: the hand-written float kernels always (plain fused multiply-adds, no
  reduced-precision matrix mode), whatever the activation dtype.  This is the whole float32 path
  and also what keeps a tensor that a checkpoint stores in 32 bits exact in a bfloat16 run.
* bfloat16 weights, up to 16 rows (decode): the hand-written skinny kernel on the matrix cores that
  streams the weight once.
* bfloat16 weights, many rows (prefill): the library product (hipBLASLt through torch), as the
  reference's engine leaves its matrix products to its tensor library
  (crates/burn-lm-llama/src/nn/attention/mha.rs:124-126).
"""
from __future__ import annotations

import torch

from ..csrc import ops

SKINNY_MAX_ROWS = 8
MFMA_SKINNY_MAX_ROWS = 16


class Runtime:
    def __init__(self, dtype=torch.bfloat16, device="cuda:0", page_size=64):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"activation dtype must be bfloat16 or float32, got {dtype}")
        self.dtype = dtype
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("burn-lm_amd runs on the GPU only (device 'cuda:N'); there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible to this process; burn-lm_amd has no CPU path")
        self.page_size = page_size
        self.ops = ops
        ops.library()  # fail now, loudly, if the kernel library cannot be had

    def empty(self, *shape, dtype=None):
        return torch.empty(*shape, dtype=dtype or self.dtype, device=self.device)

    def linear(self, x, w, out_dtype=None, out=None):
        """x [M,K] @ w[N,K]^T -> [M,N] in out_dtype (default: the activation dtype)."""
        M, K = x.shape
        N = w.shape[0]
        out_dtype = out_dtype or self.dtype
        if out is None:
            out = torch.empty(M, N, dtype=out_dtype, device=x.device)
        if w.dtype == torch.float32 or x.dtype == torch.float32:
            if M <= SKINNY_MAX_ROWS and x.dtype == w.dtype == out_dtype == torch.float32 and K % 8 == 0 \
                    and x.stride(0) % 8 == 0:
                return ops.gemv_skinny(x, w, out)
            return ops.gemm_tiled(x, w, out)
        aligned = K % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
        if M <= MFMA_SKINNY_MAX_ROWS and aligned and ops.gemv_mfma_supported(M, N, K):
            return ops.gemv_mfma(x, w, out)
        if M <= SKINNY_MAX_ROWS and aligned:
            return ops.gemv_skinny(x, w, out)
        if out_dtype == torch.bfloat16:
            return torch.matmul(x, w.t(), out=out)
        # float32 logits from bfloat16 operands with many rows: own kernel (float accumulation)
        return ops.gemm_tiled(x, w, out)

    def swiglu_linear(self, gate_up, w):
        """(silu(gate) * up) [M,K] @ w[N,K]^T for gate_up = [gate | up] of width 2K.  With few rows in
        bfloat16 the gating is fused into the product's operand load; otherwise it runs as a kernel
        of its own before the product."""
        M = gate_up.shape[0]
        N, K = w.shape
        if (gate_up.dtype == w.dtype == torch.bfloat16 and M <= MFMA_SKINNY_MAX_ROWS and K % 8 == 0
                and gate_up.stride(0) % 8 == 0 and gate_up.data_ptr() % 16 == 0 and ops.gemv_mfma_supported(M, N, K)):
            out = torch.empty(M, N, dtype=self.dtype, device=gate_up.device)
            return ops.gemv_mfma(gate_up, w, out, swiglu=True)
        act = torch.empty(M, K, dtype=gate_up.dtype, device=gate_up.device)
        ops.swiglu(gate_up, act)
        return self.linear(act, w)
