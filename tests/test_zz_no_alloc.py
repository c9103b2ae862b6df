"""dv_gather_transposed_gemv_static_f16: the entry point that allocates nothing (its split
partial sums live in a fixed array inside the library) against dv_gather_transposed_gemv_f16
with a caller-provided workspace: same kernels, so the outputs must be bit-identical; the first
call is also checked against the oracle.  Two calls in a row, the second with a smaller input,
so that what the first call left in the shared array is there when the second runs."""
import numpy as np
import pytest
import torch

from oracle import dejavu_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
REL_L2 = 1e-3


def _inputs(B, N, Z, M, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, M, generator=g).half()
    W = (torch.randn(Z, N, generator=g) * 0.02).half()
    bias = (torch.randn(N, generator=g) * 0.02).half()
    idx = torch.randperm(Z, generator=g)[:M].sort().values
    return x, W, bias, idx


def _call_pair(B, N, Z, M, seed):
    from dejavu_amd._lib import lib

    x, W, bias, idx = _inputs(B, N, Z, M, seed)
    xd, Wd, bd, idd = x.cuda(), W.cuda(), bias.cuda(), idx.cuda()
    stream = torch.cuda.current_stream().cuda_stream
    y_static = torch.full((B, N), float("nan"), dtype=torch.float16, device="cuda")
    y_ws = torch.full((B, N), float("nan"), dtype=torch.float16, device="cuda")
    nbytes = lib.dv_gather_transposed_gemv_workspace_bytes(B, N, M)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    print(f"case static scratch B={B} N={N} Z={Z} M={M} seed={seed} need={nbytes}", flush=True)
    rc = lib.dv_gather_transposed_gemv_static_f16(xd.data_ptr(), Wd.data_ptr(), N, bd.data_ptr(), idd.data_ptr(), 8,
                                                  B, N, Z, M, y_static.data_ptr(), stream)
    assert rc == 0, rc
    rc = lib.dv_gather_transposed_gemv_f16(xd.data_ptr(), Wd.data_ptr(), N, bd.data_ptr(), idd.data_ptr(), 8, B, N,
                                           Z, M, y_ws.data_ptr(), ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return (x, W, bias, idx), y_static.cpu(), y_ws.cpu()


def test_static_scratch_entry_point_matches_workspace_entry_point():
    # first call: 6 MiB of partial sums at batch 4; second call: a smaller batch, width and row count
    (x, W, bias, idx), got, want = _call_pair(4, 4096, 8192, 2048, seed=11)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "first call differs from the workspace path"
    ref = O.gather_transposed_gemv(x.numpy(), W.numpy(), idx.numpy(), bias.numpy()).astype(np.float64)
    g = got.numpy().astype(np.float64)
    assert np.abs(g - ref).max() <= MAX_ABS and np.linalg.norm(g - ref) / np.linalg.norm(ref) <= REL_L2
    (x, W, bias, idx), got, want = _call_pair(1, 1024, 2048, 520, seed=12)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "second call differs from the workspace path"
    ref = O.gather_transposed_gemv(x.numpy(), W.numpy(), idx.numpy(), bias.numpy()).astype(np.float64)
    g = got.numpy().astype(np.float64)
    assert np.abs(g - ref).max() <= MAX_ABS and np.linalg.norm(g - ref) / np.linalg.norm(ref) <= REL_L2
    # the matrix-core path (batch > 4) through the same array
    (x, W, bias, idx), got, want = _call_pair(16, 2048, 4096, 1024, seed=13)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "batch-16 call differs from the workspace path"


def test_static_scratch_entry_point_rejects_shapes_beyond_the_array():
    from dejavu_amd._lib import lib

    B, N, M = 64, 12288, 4096
    assert lib.dv_gather_transposed_gemv_workspace_bytes(B, N, M) > 8 << 20
    rc = lib.dv_gather_transposed_gemv_static_f16(0x1000, 0x1000, N, None, 0x1000, 8, B, N, 49152, M, 0x1000, None)
    assert rc == -4


def test_static_scratch_calls_on_two_streams_do_not_share_partial_sums():
    """Two calls in flight at once on two streams (each stream has its own slot of the library's array):
    both results equal the workspace entry point's; a third stream is refused with DV_ERR_UNSUPPORTED."""
    from dejavu_amd._lib import lib

    B, N, Z, M = 2, 4096, 8192, 2048
    cases = []
    for seed in (21, 22):
        x, W, bias, idx = _inputs(B, N, Z, M, seed)
        cases.append([t.cuda() for t in (x, W, bias, idx)])
    nbytes = lib.dv_gather_transposed_gemv_workspace_bytes(B, N, M)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    want = []
    for xd, Wd, bd, idd in cases:
        y = torch.empty(B, N, dtype=torch.float16, device="cuda")
        assert lib.dv_gather_transposed_gemv_f16(xd.data_ptr(), Wd.data_ptr(), N, bd.data_ptr(), idd.data_ptr(), 8, B, N,
                                                 Z, M, y.data_ptr(), ws.data_ptr(), ws.numel(),
                                                 torch.cuda.current_stream().cuda_stream) == 0
        want.append(y)
    torch.cuda.synchronize()
    # the stream the other tests of this file used holds one slot; one more stream takes the second
    streams = [torch.cuda.current_stream(), torch.cuda.Stream()]
    got = [torch.full((B, N), float("nan"), dtype=torch.float16, device="cuda") for _ in cases]
    print("case static scratch on two streams", flush=True)
    for rep in range(8):  # several rounds in flight on both streams at once
        for (xd, Wd, bd, idd), y, st in zip(cases, got, streams):
            rc = lib.dv_gather_transposed_gemv_static_f16(xd.data_ptr(), Wd.data_ptr(), N, bd.data_ptr(), idd.data_ptr(),
                                                          8, B, N, Z, M, y.data_ptr(), st.cuda_stream)
            assert rc == 0, rc
    torch.cuda.synchronize()
    for y, w in zip(got, want):
        assert torch.equal(y, w)
    third = torch.cuda.Stream()
    xd, Wd, bd, idd = cases[0]
    rc = lib.dv_gather_transposed_gemv_static_f16(xd.data_ptr(), Wd.data_ptr(), N, bd.data_ptr(), idd.data_ptr(), 8, B, N,
                                                  Z, M, got[0].data_ptr(), third.cuda_stream)
    assert rc == -2, "a third stream has no slot"
    torch.cuda.synchronize()
