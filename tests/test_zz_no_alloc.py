"""The allocation-free entry point af3_dpa_forward_static_scratch against af3_dpa_forward with a caller workspace,
through the C ABI: two calls in a row on the same GPU, the second with a smaller input (the library's scratch array
keeps the first call's contents, and the second call must not see them)."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(B, H, L, D, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(B, H, L, D, generator=g).to(torch.bfloat16).cuda() for _ in range(3)]
    bias = (torch.randn(H, L, L, generator=g) * 2).to(torch.bfloat16).cuda()
    mask = torch.rand(B, L, generator=g) < 0.85
    mask[:, 0] = True
    return q, k, v, mask.cuda(), bias


def _call(entry, q, k, v, mask, bias, workspace):
    from af3_kernels_amd import _lib, ops
    out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=q.device)
    keep = ops._lift_mask(mask, q.shape[2])
    p = ops._fill_params(q, k, v, keep, bias, out, _lib.AF3_BF16, False)
    if workspace is not None:
        p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel()
    _lib.check(entry(ctypes.byref(p), ops._stream_ptr(q.device)), "attention call")
    return out, p


def test_static_scratch_entry_point_matches_the_workspace_entry_point_on_two_calls_in_a_row(oracle):
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from af3_kernels_amd import _lib, ops
    lib = _lib.load()
    # (calls that go through scratch: a bias whose rows are not 16-byte aligned; others with so few batch rows read it in place)
    for (B, H, L, D), seed in (((18, 4, 412, 32), 5), ((3, 4, 204, 32), 6)):     # the second call is the smaller one
        q, k, v, mask, bias = _inputs(B, H, L, D, seed)
        print(f"static scratch case {(B, H, L, D)}", flush=True)
        # size of the caller workspace the ordinary entry point wants
        tmp = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        p = ops._fill_params(q, k, v, ops._lift_mask(mask, L), bias, tmp, _lib.AF3_BF16, False)
        need = lib.af3_dpa_workspace_bytes(ctypes.byref(p))
        assert 0 < need <= _lib.STATIC_SCRATCH_BYTES          # these cases do use scratch, and it fits
        ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        want, _ = _call(lib.af3_dpa_forward, q, k, v, mask, bias, ws)
        got, _ = _call(lib.af3_dpa_forward_static_scratch, q, k, v, mask, bias, None)
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))       # same kernels, same bits
        f = lambda t: t.float().cpu().numpy()
        ref = oracle.dpa_formula(f(q), f(k), f(v), mask.cpu().numpy(), f(bias))
        assert np.abs(f(got) - ref).max() <= 2e-2
    # a call that needs no scratch (one batch row: bias read in place) goes straight through
    q, k, v, mask, bias = _inputs(1, 4, 100, 32, 7)
    want, _ = _call(lib.af3_dpa_forward, q, k, v, mask, bias, None)
    got, _ = _call(lib.af3_dpa_forward_static_scratch, q, k, v, mask, bias, None)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # Under stream capture the entry point must only enqueue kernels: its host-side set-up (address of the scratch array, device
    # properties, kernel attributes) happened in the eager calls above, which is the documented order -- one call outside
    # capture first.  Replays are checked against the eager result with eager work and synchronisations in between.
    q, k, v, mask, bias = _inputs(3, 4, 204, 32, 6)
    tmp = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    p = ops._fill_params(q, k, v, ops._lift_mask(mask, 204), bias, tmp, _lib.AF3_BF16, False)
    ws = torch.empty(lib.af3_dpa_workspace_bytes(ctypes.byref(p)), dtype=torch.uint8, device=q.device)
    want, _ = _call(lib.af3_dpa_forward, q, k, v, mask, bias, ws)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got, _ = _call(lib.af3_dpa_forward_static_scratch, q, k, v, mask, bias, None)
    for i in range(3):
        got.fill_(float("nan"))
        other, _ = _call(lib.af3_dpa_forward_static_scratch, *_inputs(18, 4, 412, 32, 5), None)    # eager work that overwrites the scratch array
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"replay {i}"
