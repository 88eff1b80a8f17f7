"""The split-K entry point that allocates nothing (t5a_fwd_splitk_static: partial results in the library's
static device array) against t5a_fwd_splitk with a caller's workspace, through the raw C ABI."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def call(entry, q, k, v, o, S, workspace=None, key_lens=None):
    from turbot5_amd import _lib as L, ops
    a = L.T5ASplitKArgs()
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    for name, t in (("q_strides", q), ("k_strides", k), ("v_strides", v), ("o_strides", o)):
        setattr(a, name, (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2)))
    B, H, M, D = q.shape
    a.dtype, a.B, a.H, a.M, a.N, a.D = ops._dtype_code(q), B, H, M, k.shape[2], D
    a.num_splits, a.sm_scale = S, 1.0
    if workspace is not None:
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    if key_lens is not None:
        a.key_lens = key_lens.data_ptr()
    return getattr(L.load(), entry)(C.byref(a), ops._stream(q))


def inputs(dev, B, H, M, N, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    k = (0.5 * torch.randn(B, N, H, D, generator=g)).to(dtype).to(dev).transpose(1, 2)   # cache layout (B,N,H,D)
    v = (0.5 * torch.randn(B, N, H, D, generator=g)).to(dtype).to(dev).transpose(1, 2)
    q = (0.5 * torch.randn(B, H, M, D, generator=g)).to(dtype).to(dev)
    return q, k, v


def test_static_scratch_entry_point_equals_workspace_entry_point(gpu_device):
    from turbot5_amd import _lib as L
    from oracle import t5_basic as O
    lib = L.load()
    # two calls in a row on the same device, the second smaller: the array keeps the first call's contents
    cases = [(64, 12, 1, 8192, 64, torch.bfloat16, 16), (3, 5, 2, 700, 32, torch.float32, 7),
             (2, 4, 1, 1000, 128, torch.float16, 3)]
    for i, (B, H, M, N, D, dtype, S) in enumerate(cases):
        q, k, v = inputs(gpu_device, B, H, M, N, D, dtype, seed=400 + i)
        need = lib.t5a_splitk_workspace_bytes(B, H, M, D, S)
        assert 0 < need <= L.STATIC_SCRATCH_BYTES
        ws = torch.empty(need // 4, device=gpu_device, dtype=torch.float32)
        o_ws, o_st = torch.empty_like(q), torch.full_like(q, float("nan"))
        assert call("t5a_fwd_splitk", q, k, v, o_ws, S, workspace=ws) == 0
        before = torch.cuda.memory_allocated(gpu_device)
        assert call("t5a_fwd_splitk_static", q, k, v, o_st, S) == 0, lib.t5a_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(gpu_device) == before
        assert torch.equal(o_st, o_ws), (B, H, M, N, D)                 # same kernels, same partial layout
        want = O.dense_attention(q[:2].float().cpu(), k[:2].float().cpu(), v[:2].float().cpu(), None, False, 1.0)
        tol = 1e-4 if dtype == torch.float32 else 1e-2
        assert (o_st[:2].float().cpu() - want).abs().max().item() <= tol
    # padded memories: splits without a valid key write empty partials over whatever the array held
    B, H, M, N, D, S = 4, 6, 1, 2048, 64, 8
    q, k, v = inputs(gpu_device, B, H, M, N, D, torch.bfloat16, seed=410)
    lens = torch.tensor([2048, 100, 0, 777], dtype=torch.int32, device=gpu_device)
    ws = torch.empty(lib.t5a_splitk_workspace_bytes(B, H, M, D, S) // 4, device=gpu_device)
    o_ws, o_st = torch.empty_like(q), torch.empty_like(q)
    assert call("t5a_fwd_splitk", q, k, v, o_ws, S, workspace=ws, key_lens=lens) == 0
    assert call("t5a_fwd_splitk_static", q, k, v, o_st, S, key_lens=lens) == 0
    assert torch.equal(o_st, o_ws)
    assert (o_st[2] == 0).all()


def test_static_scratch_entry_point_rejects_what_does_not_fit(gpu_device):
    from turbot5_amd import _lib as L
    lib = L.load()
    B, H, M, N, D, S = 64, 12, 4, 4096, 64, 16
    assert lib.t5a_splitk_workspace_bytes(B, H, M, D, S) > L.STATIC_SCRATCH_BYTES
    q, k, v = inputs(gpu_device, B, H, M, N, D, torch.bfloat16, seed=420)
    o = torch.zeros_like(q)
    assert call("t5a_fwd_splitk_static", q, k, v, o, S) == -8            # T5A_ERR_WORKSPACE, nothing launched
    assert b"static scratch" in lib.t5a_last_error()
    assert (o == 0).all()


def test_python_wrapper_without_allocation(gpu_device):
    from turbot5_amd import ops
    q, k, v = inputs(gpu_device, 8, 12, 1, 4096, 64, torch.bfloat16, seed=430)
    want = ops.flash_decoding_attention(q, k, v, None, 1.0, 8)
    out = torch.empty_like(q)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(gpu_device)
    got = ops.flash_decoding_attention_static(q, k, v, out, 1.0, 8)
    assert torch.cuda.memory_allocated(gpu_device) == before and got is out
    assert torch.equal(out, want)
