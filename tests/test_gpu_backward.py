"""Backward of the dense fused-bias forward (t5a_bwd_dense behind ops.FlashAttentionBias) against torch.autograd
through the oracle's dense attention on the same seeded inputs: dq, dk, dv and the gradient of the
(num_buckets, H) table.  fp32: 1e-4 relative to the gradient's scale; bf16 / fp16: 2e-2 relative to it (the
oracle differentiates fp32 math on the rounded inputs; the fp32 kernels do the same and round only their results,
the 16-bit kernels at head_dim 64 also round the probabilities and dS to the tensors' type, as the reference does).
Reference: src/turbot5/ops/fused_bias_attention.py:397-873."""
import ctypes as C

import pytest
import torch

from oracle import t5_basic as O

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def rnd(*shape, seed=0, scale=0.5, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype)


def oracle_grads(q, k, v, table, dout, causal, sm_scale):
    """Causal attention with more queries than keys: the first M - N rows see no key.  Their output is zero and they
    have no gradient; autograd through a softmax over -inf alone gives NaN instead, so the oracle is differentiated
    on the rows that see keys (same positions: the queries end where the keys end) and the others get zeros."""
    M, N = q.shape[2], k.shape[2]
    skip = max(M - N, 0) if causal else 0
    q, k, v = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    tb = table.float().clone().requires_grad_(True) if table is not None else None
    out = O.dense_attention(q[:, :, skip:], k, v, tb, causal, sm_scale)
    out.backward(dout.float()[:, :, skip:])
    out = torch.cat([torch.zeros_like(q[:, :, :skip]), out.detach()], dim=2)
    return out, q.grad, k.grad, v.grad, (tb.grad if tb is not None else None)


def check(name, got, want, tol):
    scale = max(want.abs().max().item(), 1e-6)
    err = (got.float().cpu() - want).abs().max().item()
    assert err <= tol * scale, f"{name}: max-abs {err} against a gradient scale of {scale}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,H,M,N,D", [(2, 3, 256, 256, 64), (1, 2, 200, 333, 64), (2, 2, 130, 70, 64),
                                         (1, 2, 96, 160, 32), (1, 1, 64, 64, 16), (1, 2, 1, 300, 64)])
def test_gradients_match_autograd_through_the_oracle(gpu_device, dtype, causal, B, H, M, N, D):
    from turbot5_amd import ops
    q, k, v = rnd(B, H, M, D, seed=1, dtype=dtype), rnd(B, H, N, D, seed=2, dtype=dtype), rnd(B, H, N, D, seed=3, dtype=dtype)
    table = rnd(32, H, seed=4, scale=1.0)
    dout = rnd(B, H, M, D, seed=5, scale=1.0, dtype=dtype)
    want_o, wq, wk, wv, wt = oracle_grads(q, k, v, table, dout, causal, 1.0)
    dq, dk, dv, dt = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v, table))
    out = ops.flash_attention_with_fusing_bias(dq, dk, dv, dt, causal=causal, sm_scale=1.0)
    assert (out.float().cpu() - want_o).abs().max().item() <= (1e-4 if dtype == torch.float32 else 2e-2)
    out.backward(dout.to(gpu_device))
    tol = TOL[dtype]
    check("dq", dq.grad, wq, tol)
    check("dk", dk.grad, wk, tol)
    check("dv", dv.grad, wv, tol)
    check("dtable", dt.grad, wt, tol)
    assert dq.grad.dtype == dtype and dt.grad.dtype == torch.float32 and dq.grad.shape == q.shape


@pytest.mark.parametrize("causal", [False, True])
def test_gradients_of_strided_views_without_a_table_and_with_a_scale(gpu_device, causal):
    """(B, L, H, D) projections viewed as (B, H, L, D), as the modules hand them over; no bias table; 1/sqrt(d)."""
    from turbot5_amd import ops
    B, H, L, D = 2, 4, 192, 64
    q, k, v = (rnd(B, L, H, D, seed=10 + i).transpose(1, 2) for i in range(3))
    dout = rnd(B, L, H, D, seed=13, scale=1.0).transpose(1, 2)
    want_o, wq, wk, wv, _ = oracle_grads(q, k, v, None, dout, causal, None)
    dq, dk, dv = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    out = ops.flash_attention_with_fusing_bias(dq, dk, dv, None, causal=causal)
    out.backward(dout.to(gpu_device))
    for name, g, w in (("dq", dq.grad, wq), ("dk", dk.grad, wk), ("dv", dv.grad, wv)):
        check(name, g, w, 1e-4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("M,N", [(1024, 1024), (640, 1152), (1100, 700)])
def test_16_bit_gradients_over_long_rows(gpu_device, dtype, causal, M, N):
    """16-bit tensors at head_dim 64 run on the 16-bit matrix cores.  Rows long enough for every kind of tile of
    both passes: distances saturated on either side of the diagonal (constant bias, table gradient from tile sums),
    the band around it (bias per distance, table gradient from the sums along the tile's diagonals), tiles cut by
    the causal mask and by the ends of the tensors, several workgroups per (batch, head)."""
    from turbot5_amd import ops
    B, H, D = 1, 2, 64
    q, k, v = rnd(B, H, M, D, seed=61, dtype=dtype), rnd(B, H, N, D, seed=62, dtype=dtype), rnd(B, H, N, D, seed=63, dtype=dtype)
    table = rnd(32, H, seed=64, scale=1.0)
    dout = rnd(B, H, M, D, seed=65, scale=1.0, dtype=dtype)
    _, wq, wk, wv, wt = oracle_grads(q, k, v, table, dout, causal, 1.0)
    dq, dk, dv, dt = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v, table))
    ops.flash_attention_with_fusing_bias(dq, dk, dv, dt, causal=causal, sm_scale=1.0).backward(dout.to(gpu_device))
    for name, g, w in (("dq", dq.grad, wq), ("dk", dk.grad, wk), ("dv", dv.grad, wv), ("dtable", dt.grad, wt)):
        check(name, g, w, TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,H,M,N", [(2, 2, 256, 256), (1, 2, 200, 333), (1, 2, 700, 1100), (1, 1, 1, 300), (1, 2, 130, 70)])
def test_16_bit_gradients_at_head_dim_128(gpu_device, dtype, causal, B, H, M, N):
    """The T5-3B / 11B head shape: three passes (dq, dk, dv) over rows of 256 bytes.  fp32 tensors and fp32_math have
    no backward at this head_dim and say so."""
    from turbot5_amd import ops
    D = 128
    q, k, v = rnd(B, H, M, D, seed=81, dtype=dtype), rnd(B, H, N, D, seed=82, dtype=dtype), rnd(B, H, N, D, seed=83, dtype=dtype)
    table = rnd(32, H, seed=84, scale=1.0)
    dout = rnd(B, H, M, D, seed=85, scale=1.0, dtype=dtype)
    _, wq, wk, wv, wt = oracle_grads(q, k, v, table, dout, causal, None)
    dq, dk, dv, dt = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v, table))
    ops.flash_attention_with_fusing_bias(dq, dk, dv, dt, causal=causal).backward(dout.to(gpu_device))
    for name, g, w in (("dq", dq.grad, wq), ("dk", dk.grad, wk), ("dv", dv.grad, wv), ("dtable", dt.grad, wt)):
        check(name, g, w, TOL[dtype])


def test_head_dim_128_backward_refuses_fp32(gpu_device):
    from turbot5_amd import ops
    q, k, v = (rnd(1, 1, 64, 128, seed=86 + i).to(gpu_device).requires_grad_(True) for i in range(3))
    out = ops.flash_attention_with_fusing_bias(q, k, v, None)
    with pytest.raises(NotImplementedError, match="head_dim 128"):
        out.sum().backward()


@pytest.mark.parametrize("causal", [False, True])
def test_16_bit_gradients_on_the_fp32_matrix_cores_and_of_strided_views(gpu_device, monkeypatch, causal):
    """fp32_math: the fp32 kernels also for 16-bit tensors at head_dim 64 (they only round their results), so the two
    paths bracket each other: both within the 16-bit bar of the oracle, the fp32 one within half of it.  On
    (B, L, H, D) memory viewed as (B, H, L, D), without a table and with the default scale as well."""
    from turbot5_amd import ops
    B, H, L, D = 2, 3, 320, 64
    q, k, v = (rnd(B, L, H, D, seed=70 + i, dtype=torch.bfloat16).transpose(1, 2) for i in range(3))
    dout = rnd(B, L, H, D, seed=73, scale=1.0, dtype=torch.bfloat16).transpose(1, 2)
    table = rnd(32, H, seed=74, scale=1.0)
    for tab, scale in ((table, 1.0), (None, None)):
        _, wq, wk, wv, wt = oracle_grads(q, k, v, tab, dout, causal, scale)
        for fp32_math, tol in ((False, 2e-2), (True, 1e-2)):
            monkeypatch.setattr(ops, "BACKWARD_FP32_MATH", fp32_math)
            dq, dk, dv = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
            dt = tab.to(gpu_device).requires_grad_(True) if tab is not None else None
            ops.flash_attention_with_fusing_bias(dq, dk, dv, dt, causal=causal, sm_scale=scale).backward(dout.to(gpu_device))
            for name, g, w in (("dq", dq.grad, wq), ("dk", dk.grad, wk), ("dv", dv.grad, wv)):
                check(f"{name} fp32_math={fp32_math}", g, w, tol)
            if tab is not None:
                check(f"dtable fp32_math={fp32_math}", dt.grad, wt, tol)


def test_the_two_arithmetic_paths_agree_on_random_shapes(gpu_device, monkeypatch):
    """Seeded random shapes (M and N from 1 to 1500, either larger, causal or not, with and without a table, packed
    batches with random lengths): the 16-bit kernels against the fp32 kernels on the same inputs, which the other
    tests pin to the oracle.  Size-independent, so it also runs shapes too large for autograd on the CPU."""
    import random
    from turbot5_amd import ops
    rng = random.Random(7)

    def both(fn):
        res = []
        for fp32_math in (False, True):
            monkeypatch.setattr(ops, "BACKWARD_FP32_MATH", fp32_math)
            res.append(fn())
        return res

    for case in range(14):
        dtype = rng.choice([torch.bfloat16, torch.float16])
        causal, with_table = rng.random() < 0.5, rng.random() < 0.7
        H = rng.choice([1, 2, 3])
        if case % 3 == 2:     # packed
            lens = [rng.randint(1, 700) for _ in range(rng.randint(1, 5))]
            cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=gpu_device)
            total = sum(lens)
            q, k, v, dout = (rnd(total, H, 64, seed=100 * case + i, dtype=dtype).to(gpu_device) for i in range(4))
            shape = f"packed {lens}"
        else:
            B, M, N = rng.choice([1, 2]), rng.randint(1, 1500), rng.randint(1, 1500)
            q, dout = (rnd(B, H, M, 64, seed=100 * case + i, dtype=dtype).to(gpu_device) for i in range(2))
            k, v = (rnd(B, H, N, 64, seed=100 * case + 2 + i, dtype=dtype).to(gpu_device) for i in range(2))
            shape = f"B{B} M{M} N{N}"
        table = rnd(32, H, seed=100 * case + 9, scale=1.0).to(gpu_device) if with_table else None

        def grads():
            leaves = [t.clone().requires_grad_(True) for t in (q, k, v)] + ([table.clone().requires_grad_(True)] if with_table else [])
            tab = leaves[3] if with_table else None
            if case % 3 == 2:
                out = ops.flash_attention_with_fusing_bias_varlen(*leaves[:3], tab, cu, cu, max(lens), max(lens), causal=causal, sm_scale=1.0)
            else:
                out = ops.flash_attention_with_fusing_bias(*leaves[:3], tab, causal=causal, sm_scale=1.0)
            out.backward(dout)
            return [t.grad for t in leaves]

        fast, exact = both(grads)
        for name, g, w in zip(("dq", "dk", "dv", "dtable"), fast, exact):
            assert torch.isfinite(g).all(), (case, shape, name)
            check(f"case {case} {shape} causal={causal} {dtype} {name}", g, w.float().cpu(), 2e-2)


def test_gradients_with_prescaled_query_rows(gpu_device):
    """exact_scores="prescaled": the rows carry log2(e), the score factor of the op is ln 2 -- and so is the
    factor on dq and dk.  Differentiated through ops.prescaled_query down to the hidden states and the weight."""
    from turbot5_amd import ops
    B, H, L, D = 1, 2, 160, 64
    x = rnd(B, L, H * D, seed=20)
    w = rnd(H * D, H * D, seed=21, scale=(H * D) ** -0.5)
    k, v = rnd(B, H, L, D, seed=22), rnd(B, H, L, D, seed=23)
    table = rnd(32, H, seed=24, scale=1.0)
    dout = rnd(B, H, L, D, seed=25, scale=1.0)
    xo, wo = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    qo = (xo @ wo.T).view(B, L, H, D).transpose(1, 2)
    O.dense_attention(qo, k, v, table, False, 1.0).backward(dout)
    xd, wd = x.to(gpu_device).requires_grad_(True), w.to(gpu_device).requires_grad_(True)
    qd = ops.prescaled_query(xd, wd, torch.float32).view(B, L, H, D).transpose(1, 2)
    out = ops.flash_attention_with_fusing_bias(qd, k.to(gpu_device), v.to(gpu_device), table.to(gpu_device),
                                               sm_scale=1.0, exact_scores="prescaled")
    out.backward(dout.to(gpu_device))
    check("dx", xd.grad, xo.grad, 2e-4)
    check("dw", wd.grad, wo.grad, 2e-4)


def test_rows_without_keys_and_the_raw_entry_point(gpu_device):
    """Causal with more queries than keys: the first M - N rows see nothing, their gradient is zero and nothing is
    NaN.  Called through the C ABI with guard rows around dq, dk, dv; bad arguments are refused."""
    from turbot5_amd import _lib, ops
    B, H, M, N, D = 1, 2, 200, 120, 64
    q, k, v = rnd(B, H, M, D, seed=30), rnd(B, H, N, D, seed=31), rnd(B, H, N, D, seed=32)
    table, dout = rnd(32, H, seed=33, scale=1.0), rnd(B, H, M, D, seed=34, scale=1.0)
    _, wq, wk, wv, wt = oracle_grads(q, k, v, table, dout, True, 1.0)
    dev = [t.to(gpu_device) for t in (q, k, v, table, dout)]
    o, lse = ops.flash_attention_with_fusing_bias(*dev[:4], causal=True, sm_scale=1.0, return_lse=True)
    assert torch.isinf(lse[0, 0, :M - N]).all()
    guard = 7.0
    bufs = {n: torch.full((B, H, r + 2, D), guard, device=gpu_device) for n, r in (("dq", M), ("dk", N), ("dv", N))}
    dtab = torch.full((32, H), guard, device=gpu_device)
    lib = _lib.load()
    ws = torch.empty(int(lib.t5a_bwd_workspace_bytes(B, H, M)), dtype=torch.uint8, device=gpu_device)
    a = _lib.T5ADenseBwdArgs()
    a.q, a.k, a.v, a.o, a.dout, a.lse = (t.data_ptr() for t in (dev[0], dev[1], dev[2], o, dev[4], lse))
    a.dq, a.dk, a.dv = (bufs[n][:, :, 1:-1].data_ptr() for n in ("dq", "dk", "dv"))
    a.dtable = dtab.data_ptr()
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    for name, t in (("q_strides", dev[0]), ("k_strides", dev[1]), ("v_strides", dev[2]), ("o_strides", o),
                    ("dout_strides", dev[4]), ("dq_strides", bufs["dq"]), ("dk_strides", bufs["dk"]), ("dv_strides", bufs["dv"])):
        setattr(a, name, (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2)))
    a.dtype, a.B, a.H, a.M, a.N, a.D = _lib.T5A_F32, B, H, M, N, D
    a.causal, a.sm_scale = 1, 1.0
    a.bias.table, a.bias.table_dtype = dev[3].data_ptr(), _lib.T5A_F32
    a.bias.num_buckets, a.bias.max_distance = 32, 128
    a.bias.stride_bucket, a.bias.stride_head = dev[3].stride(0), dev[3].stride(1)
    stream = torch.cuda.current_stream(gpu_device).cuda_stream
    _lib.check(lib.t5a_bwd_dense(C.byref(a), stream))
    torch.cuda.synchronize()
    for n, w in (("dq", wq), ("dk", wk), ("dv", wv)):
        buf = bufs[n].cpu()
        assert (buf[:, :, 0] == guard).all() and (buf[:, :, -1] == guard).all(), n
        assert torch.isfinite(buf).all()
        check(n, buf[:, :, 1:-1], w, 1e-4)
    assert (bufs["dq"][:, :, 1:1 + M - N] == 0).all()
    check("dtable", dtab, wt, 1e-4)
    a.workspace_bytes = 8
    assert lib.t5a_bwd_dense(C.byref(a), stream) < 0 and b"workspace" in lib.t5a_last_error()
    a.workspace_bytes = ws.numel()
    a.D = 128
    assert lib.t5a_bwd_dense(C.byref(a), stream) < 0
    a.D = D
    a.dtable = None
    assert lib.t5a_bwd_dense(C.byref(a), stream) < 0


def test_module_trains_through_the_fused_attention(gpu_device):
    """A T5FlashAttention module in training mode: gradients reach its projections and its bias table, and agree
    with the same module differentiated through the oracle's attention."""
    from turbot5_amd import T5ATTENTION_TYPES, T5Config
    cfg = T5Config(vocab_size=32, d_model=128, d_kv=64, d_ff=256, num_layers=1, num_heads=2, dropout_rate=0.0)
    torch.manual_seed(3)
    mod = T5ATTENTION_TYPES["flash"](cfg, has_relative_attention_bias=True)
    x = torch.randn(2, 150, 128)
    sd = {n: p.detach().clone().requires_grad_(True) for n, p in mod.named_parameters()}

    def heads(t):
        return t.view(2, 150, 2, 64).transpose(1, 2)
    q, k, v = (heads(x @ sd[f"{n}.weight"].T) for n in ("q", "k", "v"))
    o = O.dense_attention(q, k, v, sd["relative_attention_bias.weight"], False, 1.0)
    (o.transpose(1, 2).reshape(2, 150, 128) @ sd["o.weight"].T).square().sum().backward()
    mod = mod.to(gpu_device).train()
    out = mod(x.to(gpu_device))[0]
    out.square().sum().backward()
    for n, p in mod.named_parameters():
        check(n, p.grad, sd[n].grad, 2e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
def test_packed_gradients_match_autograd_through_the_oracle(gpu_device, dtype, causal):
    """Backward of the packed forward (t5a_bwd_varlen; reference varlen_fused_bias_attn.py:407-868): every sequence of
    the batch against autograd through the oracle's dense attention on that sequence alone; the table's gradient is
    the sum over the sequences."""
    from turbot5_amd import ops
    H, D = 3, 64
    lens = [200, 1, 129, 64, 333]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    total = int(cu[-1])
    q, k, v = (rnd(total, H, D, seed=40 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=43, scale=1.0)
    dout = rnd(total, H, D, seed=44, scale=1.0, dtype=dtype)
    wq, wk, wv = (torch.zeros(total, H, D) for _ in range(3))
    wt = torch.zeros(32, H)
    for b, n in enumerate(lens):
        s, e = int(cu[b]), int(cu[b + 1])
        _, gq, gk, gv, gt = oracle_grads(*(t[s:e].transpose(0, 1)[None] for t in (q, k, v)), table,
                                         dout[s:e].transpose(0, 1)[None], causal, 1.0)
        wq[s:e], wk[s:e], wv[s:e] = (g[0].transpose(0, 1) for g in (gq, gk, gv))
        wt += gt
    dq, dk, dv, dt = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v, table))
    dcu = cu.to(gpu_device)
    out = ops.flash_attention_with_fusing_bias_varlen(dq, dk, dv, dt, dcu, dcu, max(lens), max(lens), causal=causal, sm_scale=1.0)
    out.backward(dout.to(gpu_device))
    tol = TOL[dtype]
    for name, g, w in (("dq", dq.grad, wq), ("dk", dk.grad, wk), ("dv", dv.grad, wv), ("dtable", dt.grad, wt)):
        check(name, g, w, tol)


@pytest.mark.parametrize("causal", [False, True])
def test_packed_gradients_at_head_dim_128(gpu_device, causal):
    """The packed backward through the head_dim-128 passes (bf16), sequence by sequence against the oracle."""
    from turbot5_amd import ops
    H, D = 2, 128
    lens = [150, 1, 260, 64]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    total = int(cu[-1])
    q, k, v = (rnd(total, H, D, seed=90 + i, dtype=torch.bfloat16) for i in range(3))
    table = rnd(32, H, seed=93, scale=1.0)
    dout = rnd(total, H, D, seed=94, scale=1.0, dtype=torch.bfloat16)
    wq, wk, wv = (torch.zeros(total, H, D) for _ in range(3))
    wt = torch.zeros(32, H)
    for b, n in enumerate(lens):
        s, e = int(cu[b]), int(cu[b + 1])
        _, gq, gk, gv, gt = oracle_grads(*(t[s:e].transpose(0, 1)[None] for t in (q, k, v)), table,
                                         dout[s:e].transpose(0, 1)[None], causal, 1.0)
        wq[s:e], wk[s:e], wv[s:e] = (g[0].transpose(0, 1) for g in (gq, gk, gv))
        wt += gt
    dq, dk, dv, dt = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v, table))
    dcu = cu.to(gpu_device)
    out = ops.flash_attention_with_fusing_bias_varlen(dq, dk, dv, dt, dcu, dcu, max(lens), max(lens), causal=causal, sm_scale=1.0)
    out.backward(dout.to(gpu_device))
    for name, g, w in (("dq", dq.grad, wq), ("dk", dk.grad, wk), ("dv", dv.grad, wv), ("dtable", dt.grad, wt)):
        check(name, g, w, 2e-2)


def test_packed_gradients_of_a_padded_batch_in_place(gpu_device):
    """A right-padded (B, L) batch run in place (cu = multiples of L, seq_lens = the lengths), keys longer than the
    queries in one call (cached decoding shape): padding rows get zero gradients, the rest matches the oracle."""
    from turbot5_amd import ops
    B, L, H, D = 3, 160, 2, 64
    lens = torch.tensor([160, 37, 100], dtype=torch.int32)
    q, k, v = (rnd(B * L, H, D, seed=50 + i) for i in range(3))
    table = rnd(32, H, seed=53, scale=1.0)
    dout = rnd(B * L, H, D, seed=54, scale=1.0)
    cu = torch.arange(0, (B + 1) * L, L, dtype=torch.int32)
    wq, wk, wv = (torch.zeros(B * L, H, D) for _ in range(3))
    wt = torch.zeros(32, H)
    for b in range(B):
        s, e = b * L, b * L + int(lens[b])
        _, gq, gk, gv, gt = oracle_grads(*(t[s:e].transpose(0, 1)[None] for t in (q, k, v)), table,
                                         dout[s:e].transpose(0, 1)[None], True, 1.0)
        wq[s:e], wk[s:e], wv[s:e] = (g[0].transpose(0, 1) for g in (gq, gk, gv))
        wt += gt
    dq, dk, dv, dt = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v, table))
    out = ops.flash_attention_with_fusing_bias_varlen(dq, dk, dv, dt, cu.to(gpu_device), cu.to(gpu_device), L, L, causal=True,
                                                      sm_scale=1.0, seq_lens_q=lens.to(gpu_device), seq_lens_k=lens.to(gpu_device))
    out.backward(dout.to(gpu_device))
    for name, g, w in (("dq", dq.grad, wq), ("dk", dk.grad, wk), ("dv", dv.grad, wv), ("dtable", dt.grad, wt)):
        assert torch.isfinite(g).all()
        check(name, g, w, 1e-4)
    pad = torch.ones(B * L, dtype=torch.bool)
    for b in range(B):
        pad[b * L:b * L + int(lens[b])] = False
    assert (dq.grad.cpu()[pad] == 0).all() and (dk.grad.cpu()[pad] == 0).all() and (dv.grad.cpu()[pad] == 0).all()


def test_encoder_stack_trains_and_forward_only_ops_say_so(gpu_device):
    """A flash encoder in training mode: the loss's gradients reach every parameter (embedding, norms, projections,
    the bias table of layer 0) and match the oracle's stack differentiated by autograd.  The sparse patterns have no
    backward kernel and refuse to be differentiated instead of dropping the graph silently."""
    from oracle import t5_model as OM
    from turbot5_amd import T5Config, T5EncoderModel, ops
    # (a smooth feed-forward activation: a ReLU gate that flips between the host's and the device's rounding of a
    # pre-activation near zero moves a weight gradient by a whole term)
    cfg = T5Config(vocab_size=64, d_model=128, d_kv=64, d_ff=256, num_layers=2, num_heads=2, dropout_rate=0.0,
                   attention_type="flash", feed_forward_proj="gated-gelu")
    torch.manual_seed(5)
    m = T5EncoderModel(cfg)
    with torch.no_grad():    # T5's initialisation makes the scores tiny (uniform attention, vanishing q / k gradients)
        for n, prm in m.named_parameters():
            if n.endswith(("SelfAttention.q.weight", "SelfAttention.k.weight")):
                prm.mul_(8.0)
            if "relative_attention_bias" in n:
                prm.copy_(torch.randn_like(prm))
    ids = torch.randint(0, 64, (2, 140), generator=torch.Generator().manual_seed(6))
    sd = {n: p.detach().clone().requires_grad_(True) for n, p in m.state_dict().items()}
    # (a loss that the final norm does not make constant: a fixed random functional of the output)
    r = rnd(2, 140, 128, seed=61, scale=1.0)
    (OM.encoder_forward(sd, cfg, ids, None, "basic") * r).sum().backward()
    m = m.to(gpu_device).train()
    (m(ids.to(gpu_device)) * r.to(gpu_device)).sum().backward()
    seen = 0
    for n, p in m.named_parameters():
        assert p.grad is not None, n
        if sd[n].grad is not None:
            # (end to end through two layers of fp32 GEMMs and norms that sum in another order than the host's: the
            # attention op itself is held to 1e-4 above)
            check(n, p.grad, sd[n].grad, 3e-3)
            seen += 1
    assert seen >= 10
    q = rnd(1, 2, 256, 64, seed=60).to(gpu_device).requires_grad_(True)
    with pytest.raises(NotImplementedError):
        ops.local_attention_with_fusing_bias(q, q, q, None, 64)
    with torch.no_grad():
        ops.local_attention_with_fusing_bias(q, q, q, None, 64)
