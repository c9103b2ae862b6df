"""Functional operators with the signatures of the reference's Triton ops,
backed by the HIP kernels in libdejavu_hip.so.

Mirrors (argument order, meaning, ``assert``-style precondition failures):
  Dejavu/src/ops/triton/gather_gemv.py           gather_gemv, gather_transposed_gemv, mlp_sparse
  Dejavu/src/ops/triton/attention_proj_sparse.py qkv_proj_sparse, out_proj_sparse,
                                                 k_cache_copy_sparse, v_cache_copy_sparse
plus the predictor / top-k pair the reference runs through nn.Linear and
torch.topk (fused_dense_sparse_dejavu.py:73-76, mha_dejavu.py:1369).

Tensors are caller-owned device tensors; results are freshly allocated; the
kernels are enqueued on ``torch.cuda.current_stream()``.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from ._lib import check, lib

_ACT = {"id": _lib.DV_ACT_ID, "relu": _lib.DV_ACT_RELU}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _idx_bytes(idx: torch.Tensor) -> int:
    assert idx.dtype in (torch.int32, torch.int64), f"index dtype must be int32 or int64, got {idx.dtype}"
    return 4 if idx.dtype == torch.int32 else 8


def _require_device(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("dejavu_amd ops run on the GPU only; got a CPU tensor (there is no CPU fallback)")


# ---------------------------------------------------------------------------
# workspace (fp32 partial sums + completion counters of the split reductions)
# ---------------------------------------------------------------------------
_workspaces: dict = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Zero-initialised per-device scratch, grown on demand.  The kernels leave
    their counters at zero, so it is only cleared when (re)allocated.  Ops that
    share it must not run concurrently on different streams."""
    key = (device.type, device.index)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


# ---------------------------------------------------------------------------
# predictor + top-k
# ---------------------------------------------------------------------------
def predictor_logits(x: torch.Tensor, fc0_weight: torch.Tensor, fc1_weight: torch.Tensor,
                     hidden: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``logits = fc1(fc0(x))`` for the bias-free low-rank predictor.

    x: (B, d) fp16, fc0_weight: (r, d), fc1_weight: (out, r) -> (B, out) fp16.
    """
    _require_device(x, fc0_weight, fc1_weight)
    assert x.dim() == 2
    B, d = x.shape
    r, d2 = fc0_weight.shape
    n_out, r2 = fc1_weight.shape
    assert d2 == d and r2 == r, "predictor weight shapes do not chain"
    assert x.dtype == fc0_weight.dtype == fc1_weight.dtype == torch.float16, "predictor runs in fp16"
    x = x.contiguous()
    if fc0_weight.stride(1) != 1:
        fc0_weight = fc0_weight.contiguous()
    if fc1_weight.stride(1) != 1:
        fc1_weight = fc1_weight.contiguous()
    if hidden is None:
        hidden = torch.empty(B, r, device=x.device, dtype=x.dtype)
    logits = torch.empty(B, n_out, device=x.device, dtype=x.dtype)
    check(lib.dv_predictor_logits_f16(_ptr(x), _ptr(fc0_weight), fc0_weight.stride(0), _ptr(fc1_weight),
                                      fc1_weight.stride(0), B, d, r, n_out, _ptr(hidden), _ptr(logits),
                                      _stream()), "dv_predictor_logits_f16")
    return logits


def topk_indices(logits: torch.Tensor, k: int, dtype: torch.dtype = torch.int64) -> torch.Tensor:
    """Indices of the k largest logits (ties to the lower index), ascending.

    logits: (n,) or (B, n) fp16; for B > 1 a column is ranked by its maximum
    over the batch.  Same set as ``logits.topk(k, sorted=False)[1]`` whenever
    that set is unique.
    """
    _require_device(logits)
    assert logits.dtype == torch.float16
    lg = logits.contiguous()
    if lg.dim() == 1:
        lg = lg.unsqueeze(0)
    assert lg.dim() == 2
    B, n = lg.shape
    assert 0 <= k <= n, f"k={k} outside [0, {n}]"
    out = torch.empty(k, device=lg.device, dtype=dtype)
    check(lib.dv_topk_f16(_ptr(lg), B, n, k, _ptr(out), _idx_bytes(out), _stream()), "dv_topk_f16")
    return out


# ---------------------------------------------------------------------------
# sparse MLP
# ---------------------------------------------------------------------------
def gather_gemv(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor,
                bias: Optional[torch.Tensor] = None, activation: str = "id") -> torch.Tensor:
    """Compute y = activation(x @ weight[idx, :].T + bias[idx]).

    x: (batch, N); weight: (Z, N); idx: (M,); bias: (Z,) -> (batch, M).
    """
    assert activation in ["id", "relu", "gelu", "gelu_approx", "squared_relu"]
    if activation not in _ACT:
        raise NotImplementedError(f"activation {activation!r}: the OPT decode path uses 'relu' / 'id' only")
    _require_device(x, weight, idx, bias)
    Z, N = weight.shape
    batch, _ = x.shape
    assert x.shape == (batch, N)
    assert batch in [1, 2, 3, 4]
    (M,) = idx.shape
    x = x.contiguous()
    if weight.stride(1) > 1:
        weight = weight.contiguous()
    assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
    assert x.dtype == torch.float16, "kernels are built for fp16"
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (Z,), "Incompatible dimensions in between weight and bias"
        assert x.dtype == bias.dtype, f"Input and bias must have the same dtype, got {x.dtype} and {bias.dtype}"
    idx = idx.contiguous()
    output = torch.empty(batch, M, device=x.device, dtype=x.dtype)
    check(lib.dv_gather_gemv_f16(_ptr(x), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(idx), _idx_bytes(idx),
                                 batch, N, Z, M, _ACT[activation], _ptr(output), _stream()), "dv_gather_gemv_f16")
    return output


def gather_transposed_gemv(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor,
                           bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Compute y = weight[idx, :]^T @ x + bias.

    x: (batch, M); weight: (Z, N); idx: (M,); bias: (N,) -> (batch, N).
    """
    _require_device(x, weight, idx, bias)
    Z, N = weight.shape
    (M,) = idx.shape
    batch, _ = x.shape
    assert x.shape == (batch, M)
    assert batch in [1, 2, 3, 4]
    x = x.contiguous()
    if weight.stride(1) > 1:
        weight = weight.contiguous()
    assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
    assert x.dtype == torch.float16, "kernels are built for fp16"
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (N,), "Incompatible dimensions in between weight and bias"
        assert x.dtype == bias.dtype, f"Input and bias must have the same dtype, got {x.dtype} and {bias.dtype}"
    idx = idx.contiguous()
    output = torch.empty(batch, N, device=x.device, dtype=x.dtype)
    nbytes = lib.dv_gather_transposed_gemv_workspace_bytes(batch, N, M)
    ws = _workspace(x.device, nbytes)
    check(lib.dv_gather_transposed_gemv_f16(_ptr(x), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(idx),
                                            _idx_bytes(idx), batch, N, Z, M, _ptr(output), _ptr(ws), ws.numel(),
                                            _stream()), "dv_gather_transposed_gemv_f16")
    return output


def mlp_sparse(x, W1, W2t, idx, bias1=None, bias2=None):
    """
    x: (batch, d)
    W1: (4d, d)
    W2t: (4d, d). This is the transpose of W2, contiguous so that gathered rows stream.
    bias1: (4d)
    bias2: (d)
    """
    x = gather_gemv(x, W1, idx, bias1, activation="relu")
    x = gather_transposed_gemv(x, W2t, idx, bias2)
    return x
