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

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import check, lib

_ACT = {"id": _lib.DV_ACT_ID, "relu": _lib.DV_ACT_RELU, "gelu": _lib.DV_ACT_GELU,
        "gelu_approx": _lib.DV_ACT_GELU_APPROX, "squared_relu": _lib.DV_ACT_SQUARED_RELU}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _idx_bytes(idx: torch.Tensor) -> int:
    assert idx.dtype in (torch.int32, torch.int64), f"index dtype must be int32 or int64, got {idx.dtype}"
    return 4 if idx.dtype == torch.int32 else 8


def _expect(ok: bool, what: str) -> None:
    """Precondition failures are ``AssertionError``s, as in the reference's wrappers."""
    if not ok:
        raise AssertionError(what)


def _same_f16(name_a: str, a: torch.Tensor, name_b: str, b: Optional[torch.Tensor]) -> None:
    if b is not None:
        _expect(a.dtype == b.dtype, f"{name_a} is {a.dtype} but {name_b} is {b.dtype}: they must agree")
    _expect(a.dtype == torch.float16, f"{name_a} is {a.dtype}: the kernels are fp16 only")


def _int32_vector(name: str, t: torch.Tensor, n: int) -> None:
    _expect(t.dtype == torch.int32 and tuple(t.shape) == (n,), f"{name} must be an int32 vector of {n} entries, "
            f"got {t.dtype} {tuple(t.shape)}")


def _require_device(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("dejavu_amd ops run on the GPU only; got a CPU tensor (there is no CPU fallback)")


# ---------------------------------------------------------------------------
# workspace (fp32 partial sums of the split reductions)
# ---------------------------------------------------------------------------
_workspaces: dict = {}
# Scratch buffers that were replaced by larger ones.  They are kept for the life of the process:
# a captured HIP graph holds the raw address of the buffer that was current when it was captured,
# so that memory must never go back to the allocator while such a graph may still be replayed.
_retired_workspaces: list = []


def _grown(cache: dict, device: torch.device, nbytes: int, floor: int) -> torch.Tensor:
    # one buffer per (device, stream): ops enqueued on different streams (the modules' side stream)
    # may run at the same time and must not share partial sums
    key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = cache.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired_workspaces.append(ws)
        ws = torch.empty(max(nbytes, floor), dtype=torch.uint8, device=device)
        cache[key] = ws
    return ws


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Scratch per device and stream, grown on demand (the kernels write every word before they read it)."""
    return _grown(_workspaces, device, nbytes, 8 << 20)


# ---------------------------------------------------------------------------
# predictor + top-k
# ---------------------------------------------------------------------------
def predictor_logits(x: torch.Tensor, fc0_weight: torch.Tensor, fc1_weight: torch.Tensor,
                     hidden: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
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
    if out is None:
        logits = torch.empty(B, n_out, device=x.device, dtype=x.dtype)
    else:
        assert out.numel() == B * n_out and out.is_contiguous() and out.dtype == x.dtype
        logits = out.view(B, n_out)
    # up to 8 rows: fixed summation order (bit-exact contract); 9..64 rows: one pass on the matrix cores
    step = 8 if B <= 8 else 64
    for b0 in range(0, B, step):
        nb = min(step, B - b0)
        nbytes = lib.dv_predictor_workspace_bytes(nb, d, r)
        ws = _workspace(x.device, nbytes) if nbytes else None
        check(lib.dv_predictor_logits_ws_f16(_ptr(x[b0:]), _ptr(fc0_weight), fc0_weight.stride(0), _ptr(fc1_weight),
                                             fc1_weight.stride(0), nb, d, r, n_out, _ptr(hidden[b0:]),
                                             _ptr(logits[b0:]), _ptr(ws), 0 if ws is None else ws.numel(), _stream()),
              "dv_predictor_logits_ws_f16")
    return logits


_topk_workspaces: dict = {}


def _topk_workspace(device: torch.device) -> torch.Tensor:
    """Histogram scratch per device and stream.  Top-k calls that share it must not overlap."""
    key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _topk_workspaces.get(key)
    if ws is None:
        ws = torch.empty(lib.dv_topk_workspace_bytes(65536) // 4, dtype=torch.int32, device=device)
        _topk_workspaces[key] = ws
    return ws


def topk_indices(logits: torch.Tensor, k: int, dtype: torch.dtype = torch.int64,
                 out: Optional[torch.Tensor] = None, single_launch: bool = False) -> torch.Tensor:
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
    if out is None:
        out = torch.empty(k, device=lg.device, dtype=dtype)
    else:
        assert out.shape == (k,) and out.is_contiguous()
    if single_launch or (n > 1024 and n % 8 != 0):
        check(lib.dv_topk_search_f16(_ptr(lg), B, n, k, _ptr(out), _idx_bytes(out), _stream()), "dv_topk_search_f16")
        return out
    ws = _topk_workspace(lg.device) if n > 1024 else None
    check(lib.dv_topk_f16(_ptr(lg), B, n, k, _ptr(out), _idx_bytes(out), _ptr(ws), 0 if ws is None else ws.numel() * 4,
                          _stream()), "dv_topk_f16")
    return out


def greedy_advance(logits: torch.Tensor, token: torch.Tensor, position: torch.Tensor, seq_pos: torch.Tensor,
                   sequences: torch.Tensor, out_index: torch.Tensor, scores: Optional[torch.Tensor] = None,
                   score_index: Optional[torch.Tensor] = None) -> None:
    """Greedy step of a batch-1 generation loop, in one launch and entirely on the device:
    ``token <- argmax(logits)`` (first index among equal values), ``sequences[0, out_index++] <-
    token``, ``position++``, ``seq_pos++``, and with ``scores`` the logits row is kept at
    ``scores[score_index++]``."""
    _require_device(logits, token, position, seq_pos, sequences, out_index, scores, score_index)
    assert logits.dtype == torch.float16 and logits.dim() == 1 and logits.is_contiguous()
    assert token.dtype == position.dtype == out_index.dtype == sequences.dtype == torch.int64
    assert seq_pos.dtype == torch.int32 and sequences.is_contiguous()
    if scores is not None:
        assert scores.dtype == torch.float16 and scores.stride(-1) == 1 and score_index.dtype == torch.int64
    check(lib.dv_greedy_advance_f16(_ptr(logits), logits.numel(), _ptr(token), _ptr(position), _ptr(seq_pos),
                                    _ptr(sequences), sequences.numel(), _ptr(out_index), _ptr(scores),
                                    0 if scores is None else scores.stride(0),
                                    0 if scores is None else scores.shape[0], _ptr(score_index), _stream()),
          "dv_greedy_advance_f16")


# ---------------------------------------------------------------------------
# sparse MLP
# ---------------------------------------------------------------------------
def gather_gemv(x: torch.Tensor, weight: torch.Tensor, idx: Optional[torch.Tensor],
                bias: Optional[torch.Tensor] = None, activation: str = "id") -> torch.Tensor:
    """Rows ``idx`` of ``weight`` applied to every row of ``x``:
    ``y[b, m] = activation(weight[idx[m]] . x[b] + bias[idx[m]])`` (the fc1 of the sparse MLP;
    interface of gather_gemv.py:198-261).

    Shapes: x (batch, N), weight (Z, N), idx (M,) int32 / int64, bias (Z,); returns (batch, M).
    ``idx=None`` takes all Z rows in order (a dense product).  batch may go up to 64 (the
    reference's kernel stops at 4; from 3 rows on the product runs on the matrix cores).
    """
    _expect(activation in ("id", "relu", "gelu", "gelu_approx", "squared_relu"), f"unknown activation {activation!r}")
    _require_device(x, weight, idx, bias)
    _expect(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1],
            f"x {tuple(x.shape)} and weight {tuple(weight.shape)} must share their last dimension")
    batch, N = x.shape
    Z = weight.shape[0]
    _expect(1 <= batch <= 64, f"batch {batch} outside 1..64")
    _same_f16("x", x, "weight", weight)
    if bias is not None:
        _expect(tuple(bias.shape) == (Z,), f"bias {tuple(bias.shape)} does not match the {Z} weight rows")
        _same_f16("x", x, "bias", bias)
        bias = bias.contiguous()
    x = x.contiguous()
    if weight.stride(1) != 1:
        weight = weight.contiguous()
    M = Z
    if idx is not None:
        idx = idx.contiguous()
        M = idx.shape[0]
    output = torch.empty(batch, M, device=x.device, dtype=x.dtype)
    nbytes = lib.dv_gather_gemv_workspace_bytes(batch, N, M)  # 0 below 17 rows
    ws = _workspace(x.device, nbytes) if nbytes else None
    check(lib.dv_gather_gemv_ws_f16(_ptr(x), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(idx),
                                    8 if idx is None else _idx_bytes(idx), batch, N, Z, M, _ACT[activation],
                                    _ptr(output), _ptr(ws), 0 if ws is None else ws.numel(), _stream()),
          "dv_gather_gemv_ws_f16")
    return output


def dense_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 activation: str = "id", out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``activation(F.linear(x, weight, bias))`` for any number of rows on the matrix cores: the dense
    products of the prompt phase.  x: (..., N) fp16 with a contiguous last dimension (rows may be
    strided after flattening); weight: (M, N); returns (..., M)."""
    _expect(activation in _ACT, f"unknown activation {activation!r}")
    _require_device(x, weight, bias, out)
    M, N = weight.shape
    assert x.shape[-1] == N and x.dtype == weight.dtype == torch.float16
    lead = x.shape[:-1]
    x2 = x.reshape(-1, N)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    if weight.stride(1) != 1:
        weight = weight.contiguous()
    rows = x2.shape[0]
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (M,) and bias.dtype == x.dtype
    if out is None:
        out = torch.empty(rows, M, device=x.device, dtype=x.dtype)
    else:
        assert out.shape == (rows, M) and out.stride(1) == 1 and out.dtype == x.dtype
    nbytes = lib.dv_dense_linear_workspace_bytes(rows, N, M)
    ws = _workspace(x.device, nbytes) if nbytes else None
    check(lib.dv_dense_linear_f16(_ptr(x2), x2.stride(0) if rows > 1 else N, _ptr(weight), weight.stride(0),
                                  _ptr(bias), rows, N, M, _ACT[activation], _ptr(out), out.stride(0) if rows > 1 else M,
                                  _ptr(ws), 0 if ws is None else ws.numel(), _stream()), "dv_dense_linear_f16")
    return out.view(*lead, M) if out.is_contiguous() else out


def dense_decode_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                        activation: str = "id") -> torch.Tensor:
    """``activation(F.linear(x, weight, bias))`` for the few rows of a decode step (1..64), streamed
    by the row kernels without a gather: the dense first block and the lm_head of a generation
    step are as bandwidth-bound as the sparse blocks.  x: (..., N) -> (..., Z)."""
    lead = x.shape[:-1]
    y = gather_gemv(x.reshape(-1, x.shape[-1]), weight, None, bias, activation)
    return y.view(*lead, weight.shape[0])


DEFERRED_REDUCE_MIN_ROWS = 3  # the matrix-core path of gather_transposed_gemv


class PendingRows:
    """The (batch, 1, N) output of a transposed product whose last step -- adding up the fp32 sums of
    its row groups -- has not run: ``add_layer_norm`` / ``add_layer_norm_window`` take it in place of
    ``hidden`` and do that step in their own launch (the fc2 of one block and LayerNorm 1 of the
    next).  ``materialize()`` runs the step alone and returns the tensor.  Shape queries answer as
    the tensor would."""

    def __init__(self, y: torch.Tensor, partial: torch.Tensor, groups: int, bias: Optional[torch.Tensor]):
        self.y, self.partial, self.groups, self.bias = y, partial, groups, bias
        self._reduced = groups == 1  # a single group stores the finished rows itself
        self.shape = torch.Size((y.shape[0], 1, y.shape[1]))
        self.dtype, self.device, self.is_cuda = y.dtype, y.device, True

    def size(self, i: Optional[int] = None):
        return self.shape if i is None else self.shape[i]

    def dim(self) -> int:
        return 3

    def numel(self) -> int:
        return self.y.numel()

    def materialize(self) -> torch.Tensor:
        if not self._reduced:
            check(lib.dv_reduce_rows_f16(_ptr(self.partial), self.groups, _ptr(self.bias), self.y.shape[0],
                                         self.y.shape[1], _ptr(self.y), _stream()), "dv_reduce_rows_f16")
            self._reduced = True
        return self.y.unsqueeze(1)


def _rows_source(hidden):
    """(partial, groups, bias, complete rows) of ``hidden`` as dv_reduce_add_layer_norm_window_f16 takes them."""
    if hidden._reduced:
        return None, 1, None, hidden.y
    return hidden.partial, hidden.groups, hidden.bias, None


def gather_transposed_gemv(x: torch.Tensor, weight: torch.Tensor, idx: torch.Tensor,
                           bias: Optional[torch.Tensor] = None, defer_reduce: bool = False):
    """Gathered rows of ``weight`` combined with the coefficients in ``x``:
    ``y[b, :] = sum_m x[b, m] * weight[idx[m], :] + bias`` (the fc2 of the sparse MLP over the
    transposed weight; interface of gather_gemv.py:572-636).

    Shapes: x (batch, M), weight (Z, N), idx (M,), bias (N,); returns (batch, N); batch 1..64.
    The split reduction has a fixed order: the result does not change from run to run.
    defer_reduce (batch >= DEFERRED_REDUCE_MIN_ROWS): returns ``PendingRows`` instead, the reduction left
    to the LayerNorm that consumes the rows.
    """
    _require_device(x, weight, idx, bias)
    _expect(x.dim() == 2 and weight.dim() == 2 and idx.dim() == 1 and x.shape[1] == idx.shape[0],
            f"x {tuple(x.shape)} needs one column per entry of idx {tuple(idx.shape)}")
    batch, M = x.shape
    Z, N = weight.shape
    _expect(1 <= batch <= 64, f"batch {batch} outside 1..64")
    _same_f16("x", x, "weight", weight)
    if bias is not None:
        _expect(tuple(bias.shape) == (N,), f"bias {tuple(bias.shape)} does not match the {N} output columns")
        _same_f16("x", x, "bias", bias)
        bias = bias.contiguous()
    x = x.contiguous()
    if weight.stride(1) != 1:
        weight = weight.contiguous()
    idx = idx.contiguous()
    output = torch.empty(batch, N, device=x.device, dtype=x.dtype)
    if defer_reduce and batch >= DEFERRED_REDUCE_MIN_ROWS and M >= 1:
        # the partial sums outlive this call: a buffer of their own, not the stream's scratch
        nbytes = lib.dv_gather_transposed_gemv_partial_workspace_bytes(batch, N, M)
        partial = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        groups = ctypes.c_int(0)
        check(lib.dv_gather_transposed_gemv_partial_f16(_ptr(x), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(idx),
                                                        _idx_bytes(idx), batch, N, Z, M, _ptr(output), _ptr(partial),
                                                        partial.numel(), ctypes.byref(groups), _stream()),
              "dv_gather_transposed_gemv_partial_f16")
        return PendingRows(output, partial, groups.value, bias)
    nbytes = lib.dv_gather_transposed_gemv_workspace_bytes(batch, N, M)
    ws = _workspace(x.device, nbytes)
    check(lib.dv_gather_transposed_gemv_f16(_ptr(x), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(idx),
                                            _idx_bytes(idx), batch, N, Z, M, _ptr(output), _ptr(ws), ws.numel(),
                                            _stream()), "dv_gather_transposed_gemv_f16")
    return output


def mlp_sparse(x, W1, W2t, idx, bias1=None, bias2=None, activation="relu"):
    """The sparse MLP on the neurons ``idx``: activation(fc1) then fc2, two gathered products
    (gather_gemv.py:647-657, where the activation is ReLU).  x (batch, d); W1 and W2t both (ffn, d),
    W2t being fc2.weight transposed so that a neuron's fc2 column is a contiguous row; bias1 (ffn,),
    bias2 (d,)."""
    hidden = gather_gemv(x, W1, idx, bias1, activation=activation)
    return gather_transposed_gemv(hidden, W2t, idx, bias2)


# ---------------------------------------------------------------------------
# head-sparse attention
# ---------------------------------------------------------------------------
def qkv_proj_sparse(x: torch.Tensor, weight: torch.Tensor, head_idx: torch.Tensor, batch_idx: torch.Tensor,
                    bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                    k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                    padding: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Head-sparse QKV projection of up to 16 window tokens (interface of
    attention_proj_sparse.py:110-190): for every listed head ``h = head_idx[i]`` and every row
    ``r = batch_idx[i, s] >= 0`` the three vectors ``y[r, t, h, :] = weight[t, h] @ x[r] + bias[t, h]``
    (t = q, k, v) are written; negative entries of ``batch_idx`` skip that (head, row) pair.

    Shapes: x (rows, hidden), rows <= 16; weight (3, nheads, head_dim, hidden); head_idx (nnz,)
    int32; batch_idx (nnz, rows) int32; bias (3, nheads, head_dim).  Returns (rows, 3, nheads,
    head_dim); what is not written is uninitialised memory, or keeps the content of ``out``.

    With ``k_cache`` / ``v_cache`` (and the int32 ``padding`` offset) the same launch also stores
    the new K / V rows at cache position ``r + padding[0]``, which is what the two cache-copy ops
    would do with ``seqlen_idx = batch_idx``.
    """
    _require_device(x, weight, head_idx, batch_idx, bias)
    _expect(weight.dim() == 4 and weight.shape[0] == 3, f"weight {tuple(weight.shape)} is not (3, nheads, head_dim, hidden)")
    _, nheads, head_dim, hidden_dim = weight.shape
    _expect(head_dim in (32, 64, 128), f"head_dim {head_dim} not in 32 / 64 / 128")
    _expect(hidden_dim % 128 == 0, f"hidden size {hidden_dim} is not a multiple of 128")
    batch_size = x.shape[0]
    _expect(tuple(x.shape) == (batch_size, hidden_dim) and batch_size <= 16,
            f"x {tuple(x.shape)} must be (rows <= 16, {hidden_dim})")
    n_active = head_idx.shape[0]
    _expect(n_active <= nheads, f"{n_active} heads listed, the layer has {nheads}")
    _int32_vector("head_idx", head_idx, n_active)
    _expect(batch_idx.dtype == torch.int32 and tuple(batch_idx.shape) == (n_active, batch_size),
            f"batch_idx must be int32 ({n_active}, {batch_size}), got {batch_idx.dtype} {tuple(batch_idx.shape)}")
    _same_f16("x", x, "weight", weight)
    if bias is not None:
        _expect(tuple(bias.shape) == (3, nheads, head_dim), f"bias {tuple(bias.shape)} is not (3, {nheads}, {head_dim})")
        _same_f16("x", x, "bias", bias)
        bias = bias.contiguous()
    x, weight, head_idx, batch_idx = x.contiguous(), weight.contiguous(), head_idx.contiguous(), batch_idx.contiguous()
    if out is None:
        out = torch.empty(batch_size, 3, nheads, head_dim, device=x.device, dtype=x.dtype)
    else:
        assert out.shape == (batch_size, 3, nheads, head_dim) and out.is_contiguous() and out.dtype == x.dtype
    S = 0
    if k_cache is not None:
        assert v_cache is not None
        _require_device(k_cache, v_cache, padding)
        S = v_cache.shape[2]
        assert v_cache.shape == (1, nheads, S, head_dim) and k_cache.shape == (1, nheads, head_dim // 8, S, 8)
        assert k_cache.is_contiguous() and v_cache.is_contiguous()
        assert k_cache.dtype == x.dtype and v_cache.dtype == x.dtype
        if padding is not None:
            assert padding.shape == (1,) and padding.dtype == torch.int32
    check(lib.dv_qkv_proj_sparse_cache_f16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(head_idx), _ptr(batch_idx),
                                           batch_size, hidden_dim, nheads, head_dim, n_active, _ptr(out),
                                           _ptr(k_cache), _ptr(v_cache), _ptr(padding), S, _stream()),
          "dv_qkv_proj_sparse_cache_f16")
    return out


def qkv_proj_batch(x: torch.Tensor, weight: torch.Tensor, head_idx: torch.Tensor,
                   bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                   k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                   positions: Optional[torch.Tensor] = None, pos_add: int = 0,
                   live: Optional[torch.Tensor] = None, use_workspace: bool = True) -> torch.Tensor:
    """QKV of the active heads for one token of each of B sequences (one shared head set), on the
    matrix cores, the weights streamed once for the whole batch; with caches the K / V rows are
    appended to sequence b's cache at ``positions[b] + pos_add`` (``positions``: int32, (B,) per
    sequence or (1,) for all; None = 0).

    :param x: (B, hidden_dim), B <= 32 (rows may be strided)
    :param weight: (3, nheads, head_dim, hidden_dim)
    :param head_idx: int32, (nnz,)
    :param live: optional int32 vector or strided column, one entry per active head: heads with a
        negative entry are skipped (back-fill passes)
    :param k_cache, v_cache: (B, nheads, head_dim / 8, S, 8), (B, nheads, S, head_dim)
    :param use_workspace: False keeps the kernel that needs no scratch memory also from 9 rows on
    :return: (B, 3, nheads, head_dim); rows of inactive / skipped heads keep the content of ``out``
    """
    _require_device(x, weight, head_idx, bias, k_cache, v_cache, positions, live)
    three, nheads, head_dim, hidden_dim = weight.shape
    assert three == 3 and head_dim in [32, 64, 128] and hidden_dim % 8 == 0
    B = x.shape[0]
    assert x.shape == (B, hidden_dim) and 1 <= B <= 32 and x.stride(1) == 1
    assert x.dtype == weight.dtype == torch.float16 and weight.is_contiguous()
    n_active = head_idx.shape[0]
    assert head_idx.dtype == torch.int32 and head_idx.is_contiguous() and n_active <= nheads
    if bias is not None:
        assert bias.shape == (3, nheads, head_dim) and bias.is_contiguous() and bias.dtype == x.dtype
    if out is None:
        out = torch.empty(B, 3, nheads, head_dim, device=x.device, dtype=x.dtype)
    else:
        assert out.shape == (B, 3, nheads, head_dim) and out.is_contiguous() and out.dtype == x.dtype
    S, per_sample = 0, 0
    if k_cache is not None:
        assert v_cache is not None
        S = v_cache.shape[2]
        assert v_cache.shape == (B, nheads, S, head_dim) and k_cache.shape == (B, nheads, head_dim // 8, S, 8)
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == v_cache.dtype == x.dtype
    if positions is not None:
        assert positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() in (1, B)
        per_sample = int(positions.numel() == B and B > 1)
    live_stride = 1
    if live is not None:
        assert live.dtype == torch.int32 and live.dim() == 1 and live.shape[0] == n_active
        live_stride = live.stride(0)
    nbytes = lib.dv_qkv_proj_batch_workspace_bytes(B, hidden_dim, n_active, head_dim) if use_workspace else 0
    ws = _workspace(x.device, nbytes) if nbytes else None
    check(lib.dv_qkv_proj_batch_f16(_ptr(x), x.stride(0), _ptr(weight), _ptr(bias), _ptr(head_idx), _ptr(live),
                                    live_stride, n_active, B, hidden_dim, nheads, head_dim, _ptr(out), _ptr(k_cache),
                                    _ptr(v_cache), _ptr(positions), per_sample, int(pos_add), S, _ptr(ws),
                                    0 if ws is None else ws.numel(), _stream()),
          "dv_qkv_proj_batch_f16")
    return out


def qkv_window_batch(x_window: torch.Tensor, weight: torch.Tensor, head_idx: torch.Tensor, batch_idx: torch.Tensor,
                     nseq: int, bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                     k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                     positions: Optional[torch.Tensor] = None, pos_add: int = 0) -> torch.Tensor:
    """QKV of the active heads for every token of a back-fill window shared by ``nseq`` sequences, in ONE
    pass over the weights (``qkv_proj_batch`` once per window token would stream them once per token).

    :param x_window: (tokens, nseq * hidden) or (tokens * nseq, hidden): LayerNorm rows of the window,
        token-major; tokens <= 16, nseq <= 32
    :param batch_idx: int32 (nnz, tokens), the tracker's output: (head i, token s) is computed when
        ``batch_idx[i, s] >= 0``
    :param positions, pos_add: token s of sequence b is cached at ``positions[b] + pos_add + s``
        (``positions``: int32, (nseq,) per sequence or (1,) for all; None = 0)
    :return: (nseq, 3, nheads, head_dim) with the rows of the newest token (s = tokens - 1); rows of
        heads that were not computed for it keep the content of ``out``
    """
    _require_device(x_window, weight, head_idx, batch_idx, bias, k_cache, v_cache, positions)
    _expect(weight.dim() == 4 and weight.shape[0] == 3, f"weight {tuple(weight.shape)} is not (3, nheads, head_dim, hidden)")
    _, nheads, head_dim, hidden_dim = weight.shape
    n_active = head_idx.shape[0]
    _int32_vector("head_idx", head_idx, n_active)
    _expect(batch_idx.dtype == torch.int32 and batch_idx.dim() == 2 and batch_idx.shape[0] == n_active
            and batch_idx.is_contiguous(), "batch_idx must be a contiguous int32 (nnz, tokens) matrix")
    tokens = batch_idx.shape[1]
    _expect(1 <= tokens <= 16 and 1 <= nseq <= 32, f"{tokens} tokens x {nseq} sequences outside 16 x 32")
    x2 = x_window.reshape(-1, hidden_dim)
    _expect(x2.shape[0] >= tokens * nseq and x2.is_contiguous(), "x_window must hold tokens * nseq contiguous rows")
    _same_f16("x_window", x2, "weight", weight)
    _expect(weight.is_contiguous() and head_idx.is_contiguous(), "weight and head_idx must be contiguous")
    if bias is not None:
        _expect(tuple(bias.shape) == (3, nheads, head_dim) and bias.is_contiguous() and bias.dtype == x2.dtype,
                f"bias {tuple(bias.shape)} is not a contiguous fp16 (3, {nheads}, {head_dim}) tensor")
    if out is None:
        out = torch.empty(nseq, 3, nheads, head_dim, device=x2.device, dtype=x2.dtype)
    else:
        _expect(tuple(out.shape) == (nseq, 3, nheads, head_dim) and out.is_contiguous() and out.dtype == x2.dtype,
                "out must be a contiguous fp16 (nseq, 3, nheads, head_dim) tensor")
    S, per_sample = 0, 0
    if k_cache is not None:
        _expect(v_cache is not None, "k_cache without v_cache")
        S = v_cache.shape[2]
        _expect(tuple(v_cache.shape) == (nseq, nheads, S, head_dim)
                and tuple(k_cache.shape) == (nseq, nheads, head_dim // 8, S, 8)
                and k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == v_cache.dtype == x2.dtype,
                "caches must be contiguous fp16 (nseq, H, hd/8, S, 8) and (nseq, H, S, hd)")
    if positions is not None:
        _expect(positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() in (1, nseq),
                "positions must be int32 with one entry, or one per sequence")
        per_sample = int(positions.numel() == nseq and nseq > 1)
    nbytes = lib.dv_qkv_window_batch_workspace_bytes(tokens, nseq, hidden_dim, n_active, head_dim)
    ws = _workspace(x2.device, nbytes) if nbytes else None
    check(lib.dv_qkv_window_batch_f16(_ptr(x2), hidden_dim, _ptr(weight), _ptr(bias), _ptr(head_idx), _ptr(batch_idx),
                                      n_active, tokens, nseq, hidden_dim, nheads, head_dim, _ptr(out), _ptr(k_cache),
                                      _ptr(v_cache), _ptr(positions), per_sample, int(pos_add), S, _ptr(ws),
                                      0 if ws is None else ws.numel(), _stream()), "dv_qkv_window_batch_f16")
    return out


def out_proj_sparse(x: torch.Tensor, weight: torch.Tensor, head_idx: torch.Tensor,
                    bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Output projection over the listed heads only (interface of attention_proj_sparse.py:274-335):
    ``y[b, n] = sum_{h in head_idx} weight[n, h, :] . x[b, h, :] + bias[n]``; the context of every
    other head is never read.

    Shapes: x (batch <= 16, nheads, head_dim); weight (hidden, nheads, head_dim), the reference's
    layout; head_idx (nnz,) int32; bias (hidden,).  Returns (batch, hidden).  ``out_proj_sparse_t``
    gives the same result from the transposed weight in one pass per batch.
    """
    _require_device(x, weight, head_idx, bias)
    _expect(weight.dim() == 3 and x.dim() == 3, "x must be (batch, nheads, head_dim), weight (hidden, nheads, head_dim)")
    hidden_dim, nheads, head_dim = weight.shape
    _expect(head_dim in (32, 64, 128), f"head_dim {head_dim} not in 32 / 64 / 128")
    _expect(hidden_dim % 128 == 0, f"hidden size {hidden_dim} is not a multiple of 128")
    batch = x.shape[0]
    _expect(tuple(x.shape) == (batch, nheads, head_dim) and batch <= 16,
            f"x {tuple(x.shape)} must be (batch <= 16, {nheads}, {head_dim})")
    n_active = head_idx.shape[0]
    _int32_vector("head_idx", head_idx, n_active)
    _same_f16("x", x, "weight", weight)
    if bias is not None:
        _expect(tuple(bias.shape) == (hidden_dim,), f"bias {tuple(bias.shape)} does not match hidden size {hidden_dim}")
        _same_f16("x", x, "bias", bias)
        bias = bias.contiguous()
    x, weight, head_idx = x.contiguous(), weight.contiguous(), head_idx.contiguous()
    output = torch.empty(batch, hidden_dim, device=x.device, dtype=x.dtype)
    check(lib.dv_out_proj_sparse_f16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(head_idx), n_active, batch, nheads,
                                     head_dim, hidden_dim, _ptr(output), _stream()), "dv_out_proj_sparse_f16")
    return output


def out_proj_sparse_t(x: torch.Tensor, weight_t: torch.Tensor, head_idx: torch.Tensor,
                      bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Same result as ``out_proj_sparse`` from the transposed weight.

    :param x: (batch, nheads, head_dim)
    :param weight_t: (nheads * head_dim, hidden_dim) = out_proj.weight.t().contiguous(); the rows
        of an active head are one contiguous block
    """
    _require_device(x, weight_t, head_idx, bias)
    batch, nheads, head_dim = x.shape
    rows, hidden_dim = weight_t.shape
    assert rows == nheads * head_dim
    assert head_idx.dtype == torch.int32
    assert 1 <= batch <= 64
    n_active = head_idx.shape[0]
    x = x.contiguous()
    if weight_t.stride(1) != 1:
        weight_t = weight_t.contiguous()
    assert x.dtype == weight_t.dtype == torch.float16
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (hidden_dim,)
    head_idx = head_idx.contiguous()
    output = torch.empty(batch, hidden_dim, device=x.device, dtype=x.dtype)
    nbytes = lib.dv_out_proj_sparse_t_workspace_bytes(batch, hidden_dim, n_active, head_dim)
    ws = _workspace(x.device, nbytes)
    check(lib.dv_out_proj_sparse_t_f16(_ptr(x), _ptr(weight_t), weight_t.stride(0), _ptr(bias), _ptr(head_idx),
                                       n_active, batch, nheads, head_dim, hidden_dim, _ptr(output), _ptr(ws),
                                       ws.numel(), _stream()), "dv_out_proj_sparse_t_f16")
    return output


OUT_PROJ_LN_MIN_ROWS = 3  # the matrix-core path of out_proj_sparse_t


def out_proj_sparse_t_add_layer_norm(x: torch.Tensor, weight_t: torch.Tensor, head_idx: torch.Tensor,
                                     bias: Optional[torch.Tensor], residual: Optional[torch.Tensor],
                                     ln_weight: torch.Tensor, ln_bias: torch.Tensor, eps: float):
    """``add_layer_norm(out_proj_sparse_t(x, ...), residual, ...)`` for 3..64 rows with the split
    reduction of the projection and the LayerNorm in one launch.  Returns (normed, residual_out), both
    (batch, hidden_dim); same bits as the two ops."""
    _require_device(x, weight_t, head_idx, bias, residual, ln_weight, ln_bias)
    batch, nheads, head_dim = x.shape
    rows, hidden_dim = weight_t.shape
    assert rows == nheads * head_dim and head_idx.dtype == torch.int32
    assert OUT_PROJ_LN_MIN_ROWS <= batch <= 64
    assert x.dtype == weight_t.dtype == ln_weight.dtype == ln_bias.dtype == torch.float16
    n_active = head_idx.shape[0]
    x = x.contiguous()
    if weight_t.stride(1) != 1:
        weight_t = weight_t.contiguous()
    if bias is not None:
        bias = bias.contiguous()
    if residual is not None:
        residual = residual.contiguous()
        assert residual.numel() == batch * hidden_dim and residual.dtype == torch.float16
    head_idx = head_idx.contiguous()
    normed = torch.empty(batch, hidden_dim, device=x.device, dtype=x.dtype)
    r_out = torch.empty(batch, hidden_dim, device=x.device, dtype=x.dtype)
    nbytes = lib.dv_out_proj_sparse_t_ln_workspace_bytes(batch, n_active, head_dim, hidden_dim)
    ws = _workspace(x.device, nbytes)
    check(lib.dv_out_proj_sparse_t_ln_f16(_ptr(x), _ptr(weight_t), weight_t.stride(0), _ptr(bias), _ptr(head_idx),
                                          n_active, batch, nheads, head_dim, hidden_dim, _ptr(residual),
                                          _ptr(ln_weight.contiguous()), _ptr(ln_bias.contiguous()), float(eps),
                                          _ptr(normed), _ptr(r_out), _ptr(ws), ws.numel(), _stream()),
          "dv_out_proj_sparse_t_ln_f16")
    return normed, r_out


def _cache_copy(k, v, k_cache, v_cache, head_idx, seqlen_idx, padding):
    src = k if k is not None else v
    _require_device(src, k_cache, v_cache, head_idx, seqlen_idx, padding)
    _expect(src.dim() == 3, "k / v must be (tokens, nheads, head_dim)")
    nnz_seqlen, nheads, head_dim = src.shape
    _expect(head_dim in (32, 64, 128), f"head_dim {head_dim} not in 32 / 64 / 128")
    _expect(nnz_seqlen <= 16, f"{nnz_seqlen} tokens: a back-fill window holds at most 16")
    _expect(src.stride(2) == 1 and src.stride(1) == head_dim, "the heads of a k / v row must be contiguous")
    n_active = head_idx.shape[0]
    _expect(n_active <= nheads, f"{n_active} heads listed, the layer has {nheads}")
    _int32_vector("head_idx", head_idx, n_active)
    _expect(seqlen_idx.dtype == torch.int32 and tuple(seqlen_idx.shape) == (n_active, nnz_seqlen),
            f"seqlen_idx must be int32 ({n_active}, {nnz_seqlen}), got {seqlen_idx.dtype} {tuple(seqlen_idx.shape)}")
    if padding is not None:
        _int32_vector("padding", padding, 1)
    head_idx, seqlen_idx = head_idx.contiguous(), seqlen_idx.contiguous()
    seqlen = 0
    if k_cache is not None:
        _same_f16("k", k, "k_cache", k_cache)
        seqlen = k_cache.shape[3]
        _expect(tuple(k_cache.shape) == (1, nheads, head_dim // 8, seqlen, 8) and k_cache.is_contiguous(),
                f"k_cache {tuple(k_cache.shape)} is not a contiguous (1, {nheads}, {head_dim // 8}, S, 8) tensor")
    if v_cache is not None:
        _same_f16("v", v, "v_cache", v_cache)
        seqlen = v_cache.shape[2]
        _expect(tuple(v_cache.shape) == (1, nheads, seqlen, head_dim) and v_cache.is_contiguous(),
                f"v_cache {tuple(v_cache.shape)} is not a contiguous (1, {nheads}, S, {head_dim}) tensor")
    if k is not None and v is not None:
        _expect(k.stride(0) == v.stride(0), "k and v must have the same row stride")
    check(lib.dv_kv_cache_copy_sparse_f16(_ptr(k), _ptr(v), src.stride(0), nnz_seqlen, _ptr(k_cache), _ptr(v_cache),
                                          _ptr(head_idx), _ptr(seqlen_idx), n_active, nnz_seqlen, _ptr(padding),
                                          nheads, head_dim, seqlen, _stream()), "dv_kv_cache_copy_sparse_f16")


def k_cache_copy_sparse(k: torch.Tensor, k_cache: torch.Tensor, head_idx: torch.Tensor, seqlen_idx: torch.Tensor,
                        padding: torch.Tensor = None) -> None:
    """Stores window tokens' K rows of the listed heads into the packed key cache (interface of
    attention_proj_sparse.py:525-590): for ``h = head_idx[i]`` and ``s = seqlen_idx[i, j] >= 0``,
    ``k_cache[0, h, c // 8, s + padding[0], c % 8] = k[s, h, c]``.  k (tokens <= 16, nheads,
    head_dim); k_cache (1, nheads, head_dim / 8, S, 8); head_idx (nnz,), seqlen_idx (nnz, tokens)
    and padding (1,) int32."""
    _cache_copy(k, None, k_cache, None, head_idx, seqlen_idx, padding)


def v_cache_copy_sparse(v: torch.Tensor, v_cache: torch.Tensor, head_idx: torch.Tensor, seqlen_idx: torch.Tensor,
                        padding: torch.Tensor = None) -> None:
    """The value-cache counterpart of ``k_cache_copy_sparse`` (attention_proj_sparse.py:396-459):
    ``v_cache[0, h, s + padding[0], :] = v[s, h, :]``; v_cache is (1, nheads, S, head_dim)."""
    _cache_copy(None, v, None, v_cache, head_idx, seqlen_idx, padding)


def kv_cache_copy_sparse(k, v, k_cache, v_cache, head_idx, seqlen_idx, padding=None) -> None:
    """Both cache copies in one launch."""
    _cache_copy(k, v, k_cache, v_cache, head_idx, seqlen_idx, padding)


def require_no_rotary(rotary_emb_dim: int) -> None:
    """The one place where a rotary embedding is turned down: OPT uses learned positions, and the
    rotation that ``ft_attention.single_query_attention`` applies to q and k for ``rotary_emb_dim > 0``
    (mha_dejavu.py:1439-1456) is not built here."""
    if rotary_emb_dim != 0:
        raise NotImplementedError(f"rotary_emb_dim = {rotary_emb_dim}: rotary position embedding is not built "
                                  "(OPT uses learned positions)")


def single_query_attention(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                           k_cache: torch.Tensor, v_cache: torch.Tensor,
                           lengths_per_sample: Optional[torch.Tensor], timestep: int, rotary_emb_dim: int = 0,
                           head_idx: Optional[torch.Tensor] = None, softmax_scale: Optional[float] = None,
                           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Decode attention with the call shape of ``ft_attention.single_query_attention``.

    q, k, v: (B, H, hd) of the newest token (last dim contiguous); k_cache (B, H, hd/8, S, 8);
    v_cache (B, H, S, hd).  k, v are written at position ``timestep`` (``lengths_per_sample[b]``
    when given) and positions up to and including it are attended.  Pass ``k = v = None`` when the
    caches already hold the newest token.  With ``head_idx`` (int32) only those heads are touched
    and only their rows of the (B, H, hd) result are written.
    """
    _require_device(q, k, v, k_cache, v_cache, lengths_per_sample, head_idx)
    require_no_rotary(rotary_emb_dim)
    B, H, hd = q.shape
    S = v_cache.shape[2]
    assert hd in [32, 64, 128], "the decode attention kernels are built for head_dim 32, 64 and 128"
    assert q.dtype == torch.float16 and k_cache.dtype == torch.float16 and v_cache.dtype == torch.float16
    assert v_cache.shape == (B, H, S, hd) and k_cache.shape == (B, H, hd // 8, S, 8)
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert q.stride(2) == 1 and q.stride(1) == hd
    assert 0 <= timestep < S
    nheads = 0
    if head_idx is not None:
        assert head_idx.dtype == torch.int32
        head_idx = head_idx.contiguous()
        nheads = head_idx.shape[0]
    if lengths_per_sample is not None:
        assert lengths_per_sample.dtype == torch.int32 and lengths_per_sample.shape == (B,)
    if k is not None:
        assert v is not None and k.shape == (B, H, hd) and v.shape == (B, H, hd)
        assert k.stride(2) == 1 and k.stride(1) == hd and v.stride(2) == 1 and v.stride(1) == hd
        assert k.stride(0) == v.stride(0)
        check(lib.dv_kv_append_f16(_ptr(k), _ptr(v), k.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(head_idx),
                                   nheads, _ptr(lengths_per_sample), timestep, B, H, hd, S, _stream()),
              "dv_kv_append_f16")
    if out is None:
        out = torch.empty(B, H, hd, device=q.device, dtype=q.dtype)
    n_len = S if lengths_per_sample is not None else timestep + 1
    scale = float(hd ** -0.5 if softmax_scale is None else softmax_scale)
    n_heads_ws = nheads if head_idx is not None else H
    nbytes = lib.dv_decode_attention_workspace_bytes(B, n_heads_ws, n_len, hd)
    ws = _attn_workspace(q.device, nbytes)
    check(lib.dv_decode_attention_f16(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(head_idx), nheads,
                                      _ptr(lengths_per_sample), n_len, B, H, hd, S, scale, _ptr(out), out.stride(0),
                                      _ptr(ws), ws.numel(), _stream()), "dv_decode_attention_f16")
    return out


def prefill_attention(qkv: torch.Tensor, k_cache: Optional[torch.Tensor] = None,
                      v_cache: Optional[torch.Tensor] = None, pos0: int = 0,
                      softmax_scale: Optional[float] = None) -> torch.Tensor:
    """Causal attention over the prompt; with caches, the prompt's K / V rows are also written to
    positions ``pos0 .. pos0 + T - 1`` of the (packed) decode caches by the same launch.

    qkv: (B, T, 3, H, hd) fp16 contiguous -> context (B, T, H * hd).
    k_cache (B, H, hd / 8, S, 8), v_cache (B, H, S, hd).
    """
    _require_device(qkv, k_cache, v_cache)
    B, T, three, H, hd = qkv.shape
    assert three == 3 and hd in [64, 128], "the prompt attention kernel is built for head_dim 64 and 128"
    assert qkv.dtype == torch.float16 and qkv.is_contiguous()
    S = 0
    if k_cache is not None:
        assert v_cache is not None
        S = v_cache.shape[2]
        assert v_cache.shape == (B, H, S, hd) and k_cache.shape == (B, H, hd // 8, S, 8)
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == v_cache.dtype == qkv.dtype
        assert 0 <= pos0 and pos0 + T <= S
    ctx = torch.empty(B, T, H * hd, device=qkv.device, dtype=qkv.dtype)
    scale = float(hd ** -0.5 if softmax_scale is None else softmax_scale)
    check(lib.dv_prefill_attention_f16(_ptr(qkv), B, T, H, hd, scale, _ptr(ctx), _ptr(k_cache), _ptr(v_cache),
                                       int(pos0), S, _stream()), "dv_prefill_attention_f16")
    return ctx


_attn_workspaces: dict = {}


def _attn_workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    return _grown(_attn_workspaces, device, nbytes, 4 << 20)


# ---------------------------------------------------------------------------
# block glue
# ---------------------------------------------------------------------------
def add_layer_norm(hidden: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor,
                   bias: torch.Tensor, eps: float = 1e-5):
    """``residual_out = hidden + residual`` (fp16) and ``LayerNorm(residual_out)``.

    hidden / residual: (..., d) fp16.  Returns (normed, residual_out), both shaped like hidden.
    ``hidden`` may be ``PendingRows``: its reduction then runs in the same launch.
    """
    if isinstance(hidden, PendingRows):
        return _reduce_add_layer_norm(hidden, residual, weight, bias, eps, None)
    _require_device(hidden, residual, weight, bias)
    assert hidden.dtype == torch.float16 and weight.dtype == torch.float16 and bias.dtype == torch.float16
    d = hidden.shape[-1]
    assert weight.shape == (d,) and bias.shape == (d,)
    hidden = hidden.contiguous()
    if residual is not None:
        assert residual.shape == hidden.shape and residual.dtype == hidden.dtype
        residual = residual.contiguous()
    rows = hidden.numel() // d
    y = torch.empty_like(hidden)
    r_out = torch.empty_like(hidden)
    check(lib.dv_add_layer_norm_f16(_ptr(hidden), _ptr(residual), _ptr(weight.contiguous()), _ptr(bias.contiguous()),
                                    float(eps), rows, d, _ptr(y), _ptr(r_out), _stream()), "dv_add_layer_norm_f16")
    return y, r_out


def add_layer_norm_window(hidden: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor,
                          bias: torch.Tensor, eps: float, x_cache_row: torch.Tensor, tracker: torch.Tensor,
                          head_idx: torch.Tensor, counter: int, flush: bool, batch_idx: torch.Tensor):
    """``add_layer_norm`` for the rows of B sequences that share a back-fill window, with the window
    step of the same position in the same launch: the normalised rows also go to ``x_cache_row``
    ((B * d,) row ``counter`` of the window buffer) and the tracker hands out ``batch_idx``
    ((nnz, counter + 1) int32; see ``dv_window_step_f16``).  Returns (normed, residual_out).
    ``hidden`` may be ``PendingRows``: its reduction then runs in the same launch."""
    if isinstance(hidden, PendingRows):
        return _reduce_add_layer_norm(hidden, residual, weight, bias, eps,
                                      (x_cache_row, tracker, head_idx, counter, flush, batch_idx))
    _require_device(hidden, residual, weight, bias, x_cache_row, tracker, head_idx, batch_idx)
    assert hidden.dtype == torch.float16 and weight.dtype == torch.float16 and bias.dtype == torch.float16
    d = hidden.shape[-1]
    hidden = hidden.contiguous()
    rows = hidden.numel() // d
    if residual is not None:
        assert residual.shape == hidden.shape and residual.dtype == hidden.dtype
        residual = residual.contiguous()
    assert x_cache_row.dtype == torch.float16 and x_cache_row.is_contiguous() and x_cache_row.numel() == rows * d
    assert tracker.dtype == torch.int32 and head_idx.dtype == torch.int32 and batch_idx.dtype == torch.int32
    assert tracker.is_contiguous() and batch_idx.is_contiguous() and head_idx.is_contiguous()
    H = tracker.shape[0]
    nnz = head_idx.shape[0]
    assert batch_idx.numel() >= nnz * (counter + 1)
    y = torch.empty_like(hidden)
    r_out = torch.empty_like(hidden)
    check(lib.dv_add_layer_norm_window_f16(_ptr(hidden), _ptr(residual), _ptr(weight.contiguous()),
                                           _ptr(bias.contiguous()), float(eps), rows, d, _ptr(y), _ptr(r_out),
                                           _ptr(x_cache_row), _ptr(tracker), _ptr(head_idx), nnz, H, int(counter),
                                           int(flush), _ptr(batch_idx), _stream()),
          "dv_add_layer_norm_window_f16")
    return y, r_out


def _reduce_add_layer_norm(hidden: PendingRows, residual: Optional[torch.Tensor], weight: torch.Tensor,
                           bias: torch.Tensor, eps: float, window):
    """add_layer_norm / add_layer_norm_window of rows whose split reduction is still to run."""
    _require_device(residual, weight, bias)
    rows, d = hidden.y.shape
    assert weight.dtype == torch.float16 and bias.dtype == torch.float16 and weight.shape == (d,) and bias.shape == (d,)
    if residual is not None:
        assert residual.numel() == rows * d and residual.dtype == torch.float16
        residual = residual.contiguous()
    partial, groups, pbias, complete = _rows_source(hidden)
    y = torch.empty(rows, 1, d, dtype=torch.float16, device=hidden.device)
    r_out = torch.empty_like(y)
    if window is None:
        x_cache_row = tracker = head_idx = batch_idx = None
        nnz = H = counter = flush = 0
    else:
        x_cache_row, tracker, head_idx, counter, flush, batch_idx = window
        _require_device(x_cache_row, tracker, head_idx, batch_idx)
        assert x_cache_row.dtype == torch.float16 and x_cache_row.is_contiguous() and x_cache_row.numel() == rows * d
        assert tracker.dtype == torch.int32 and head_idx.dtype == torch.int32 and batch_idx.dtype == torch.int32
        assert tracker.is_contiguous() and batch_idx.is_contiguous() and head_idx.is_contiguous()
        H, nnz = tracker.shape[0], head_idx.shape[0]
        assert batch_idx.numel() >= nnz * (counter + 1)
    check(lib.dv_reduce_add_layer_norm_window_f16(_ptr(partial), groups, _ptr(pbias), _ptr(complete), _ptr(residual),
                                                  _ptr(weight.contiguous()), _ptr(bias.contiguous()), float(eps), rows,
                                                  d, _ptr(y), _ptr(r_out), _ptr(x_cache_row), _ptr(tracker),
                                                  _ptr(head_idx), nnz, H, int(counter), int(flush), _ptr(batch_idx),
                                                  _stream()), "dv_reduce_add_layer_norm_window_f16")
    return y, r_out


def add_ln_parts(hidden: torch.Tensor, residual: Optional[torch.Tensor]):
    """First half of ``add_layer_norm`` for ONE row when the consumer of the row normalises it itself:
    ``r = hidden + residual`` (fp16) and the statistics pairs of r's 64-element parts (float32,
    (ceil(d / 64), 2): sum, sum of squared deviations from the part's mean).  Returns (r, parts)."""
    _require_device(hidden, residual)
    assert hidden.dtype == torch.float16
    d = hidden.shape[-1]
    assert hidden.numel() == d, "one row"
    hidden = hidden.contiguous()
    if residual is not None:
        assert residual.shape == hidden.shape and residual.dtype == hidden.dtype
        residual = residual.contiguous()
    r_out = torch.empty_like(hidden)
    parts = torch.empty((d + 63) // 64, 2, dtype=torch.float32, device=hidden.device)
    check(lib.dv_add_ln_parts_f16(_ptr(hidden), _ptr(residual), d, _ptr(r_out), _ptr(parts), _stream()),
          "dv_add_ln_parts_f16")
    return r_out, parts


def ln_qkv_proj_sparse(r: torch.Tensor, parts: torch.Tensor, ln_weight: torch.Tensor, ln_bias: torch.Tensor,
                       eps: float, x_cache: torch.Tensor, token: int, weight: torch.Tensor, head_idx: torch.Tensor,
                       batch_idx: torch.Tensor, bias: Optional[torch.Tensor] = None,
                       out: Optional[torch.Tensor] = None, k_cache: Optional[torch.Tensor] = None,
                       v_cache: Optional[torch.Tensor] = None, padding: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``qkv_proj_sparse`` for window position ``token`` with the LayerNorm of the newest row folded
    in: ``r`` / ``parts`` come from ``add_ln_parts``; the QKV workgroups normalise the row themselves
    (``ln_weight``, ``ln_bias``, ``eps``), the normalised row lands in ``x_cache[token]`` and rows
    ``0 .. token - 1`` are read from ``x_cache`` ((16, hidden) window buffer).  Same bits as
    ``add_layer_norm`` followed by ``qkv_proj_sparse(x_cache[:token + 1], ...)``.  batch_idx:
    (nnz, token + 1) int32; with token == 0 every listed head is computed."""
    _require_device(r, parts, ln_weight, ln_bias, x_cache, weight, head_idx, batch_idx, bias)
    _, nheads, head_dim, hidden_dim = weight.shape
    nb = token + 1
    _expect(head_dim in (64, 128), f"head_dim {head_dim} not 64 / 128")
    _expect(r.numel() == hidden_dim and r.dtype == torch.float16, "r must be one fp16 row")
    _expect(parts.dtype == torch.float32 and tuple(parts.shape) == ((hidden_dim + 63) // 64, 2), "parts from add_ln_parts")
    _expect(tuple(x_cache.shape) == (16, hidden_dim) and x_cache.is_contiguous(), "x_cache must be the (16, hidden) window buffer")
    n_active = head_idx.shape[0]
    _int32_vector("head_idx", head_idx, n_active)
    _expect(batch_idx.dtype == torch.int32 and tuple(batch_idx.shape) == (n_active, nb),
            f"batch_idx must be int32 ({n_active}, {nb})")
    if bias is not None:
        bias = bias.contiguous()
    r, weight, head_idx, batch_idx = r.contiguous(), weight.contiguous(), head_idx.contiguous(), batch_idx.contiguous()
    if out is None:
        out = torch.empty(nb, 3, nheads, head_dim, device=r.device, dtype=r.dtype)
    else:
        assert out.shape == (nb, 3, nheads, head_dim) and out.is_contiguous() and out.dtype == r.dtype
    S = 0
    if k_cache is not None:
        assert v_cache is not None
        _require_device(k_cache, v_cache, padding)
        S = v_cache.shape[2]
        assert v_cache.shape == (1, nheads, S, head_dim) and k_cache.shape == (1, nheads, head_dim // 8, S, 8)
        assert k_cache.is_contiguous() and v_cache.is_contiguous()
    check(lib.dv_ln_qkv_proj_sparse_cache_f16(_ptr(r), _ptr(parts), _ptr(ln_weight.contiguous()),
                                              _ptr(ln_bias.contiguous()), float(eps), _ptr(x_cache), token,
                                              _ptr(weight), _ptr(bias), _ptr(head_idx), _ptr(batch_idx), nb, hidden_dim,
                                              nheads, head_dim, n_active, _ptr(out), _ptr(k_cache), _ptr(v_cache),
                                              _ptr(padding), S, _stream()), "dv_ln_qkv_proj_sparse_cache_f16")
    return out


def attention_out_proj(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, head_idx: torch.Tensor,
                       timestep: int, weight_t: torch.Tensor, bias: Optional[torch.Tensor] = None,
                       lengths_per_sample: Optional[torch.Tensor] = None,
                       softmax_scale: Optional[float] = None) -> torch.Tensor:
    """``out_proj_sparse_t(single_query_attention(q, ...), weight_t, head_idx, bias)`` in two launches,
    without writing the context vector: the out_proj kernel merges the attention splits itself.

    q: (B, H, hd); caches already hold the newest token; weight_t: (H*hd, d).  Returns (B, d).
    """
    _require_device(q, k_cache, v_cache, head_idx, weight_t, bias, lengths_per_sample)
    B, H, hd = q.shape
    S = v_cache.shape[2]
    rows, N = weight_t.shape
    assert rows == H * hd and head_idx.dtype == torch.int32 and B in [1, 2, 3, 4]
    assert q.dtype == k_cache.dtype == v_cache.dtype == weight_t.dtype == torch.float16
    assert v_cache.shape == (B, H, S, hd) and k_cache.shape == (B, H, hd // 8, S, 8)
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and q.stride(2) == 1 and q.stride(1) == hd
    assert 0 <= timestep < S
    if weight_t.stride(1) != 1:
        weight_t = weight_t.contiguous()
    head_idx = head_idx.contiguous()
    nheads = head_idx.shape[0]
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (N,)
    if lengths_per_sample is not None:
        assert lengths_per_sample.dtype == torch.int32 and lengths_per_sample.shape == (B,)
    n_len = S if lengths_per_sample is not None else timestep + 1
    scale = float(hd ** -0.5 if softmax_scale is None else softmax_scale)
    out = torch.empty(B, N, device=q.device, dtype=q.dtype)
    nbytes = lib.dv_attention_out_proj_workspace_bytes(B, nheads, n_len, hd, N)
    ws = _workspace(q.device, nbytes)
    check(lib.dv_attention_out_proj_f16(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(head_idx), nheads,
                                        _ptr(lengths_per_sample), n_len, B, H, hd, S, scale, _ptr(weight_t),
                                        weight_t.stride(0), _ptr(bias), N, _ptr(out), _ptr(ws), ws.numel(),
                                        _stream()), "dv_attention_out_proj_f16")
    return out


def attention_out_proj_rows(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, head_idx: torch.Tensor,
                            timestep: int, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                            lengths_per_sample: Optional[torch.Tensor] = None,
                            softmax_scale: Optional[float] = None,
                            residual: Optional[torch.Tensor] = None):
    """``out_proj_sparse(single_query_attention(q, ...), weight, head_idx, bias)`` for one sequence in two
    launches, weight in out_proj.weight's own layout (d, H, hd): the out_proj kernel merges the attention
    splits itself and finishes every output row inside one wavefront (no split reduction).

    q: (1, H, hd); caches already hold the newest token.  Returns y (1, d); with ``residual`` (1, d) or (d,)
    returns (y, fp16(y + residual)), the residual stream advanced in the same launch.
    """
    _require_device(q, k_cache, v_cache, head_idx, weight, bias, lengths_per_sample, residual)
    B, H, hd = q.shape
    S = v_cache.shape[2]
    N = weight.shape[0]
    assert B == 1 and weight.numel() == N * H * hd and weight.is_contiguous()
    assert head_idx.dtype == torch.int32 and head_idx.numel() >= 1
    assert q.dtype == k_cache.dtype == v_cache.dtype == weight.dtype == torch.float16
    assert v_cache.shape == (B, H, S, hd) and k_cache.shape == (B, H, hd // 8, S, 8)
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and q.stride(2) == 1 and q.stride(1) == hd
    assert 0 <= timestep < S
    head_idx = head_idx.contiguous()
    nheads = head_idx.shape[0]
    if bias is not None:
        bias = bias.contiguous()
        assert bias.shape == (N,)
    if lengths_per_sample is not None:
        assert lengths_per_sample.dtype == torch.int32 and lengths_per_sample.shape == (B,)
    n_len = S if lengths_per_sample is not None else timestep + 1
    scale = float(hd ** -0.5 if softmax_scale is None else softmax_scale)
    out = torch.empty(B, N, device=q.device, dtype=q.dtype)
    res_out = None
    if residual is not None:
        residual = residual.contiguous()
        assert residual.numel() == N and residual.dtype == torch.float16
        res_out = torch.empty_like(residual)
    nbytes = lib.dv_decode_attention_workspace_bytes(1, nheads, n_len, hd)
    ws = _attn_workspace(q.device, nbytes)
    check(lib.dv_attention_out_proj_rows_f16(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(head_idx),
                                             nheads, _ptr(lengths_per_sample), n_len, H, hd, S, scale, _ptr(weight),
                                             _ptr(bias), N, _ptr(out), _ptr(residual), _ptr(res_out), _ptr(ws),
                                             ws.numel(), _stream()), "dv_attention_out_proj_rows_f16")
    return out if residual is None else (out, res_out)
