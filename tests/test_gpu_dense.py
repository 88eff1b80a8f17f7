"""GPU parity of the dense and packed fused-bias forwards against the CPU oracle.

Tolerances (max-abs): bf16/fp16 2e-2, fp32 1e-4 -- the bars the build was given.
The oracle runs fp32 math on the same (already rounded) inputs.
"""
import numpy as np
import pytest
import torch

from oracle import t5_basic as O

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 2e-2, torch.float32: 1e-4}


def rnd(*shape, seed=0, scale=0.5, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype)


def run_dense(dev, B, H, M, N, D, dtype, causal, bias=True, sm_scale=1.0, seed=0, nb=32, md=128, blhd=False):
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    if blhd:   # (B,H,L,D) views of (B,L,H,D) memory, as the attention modules produce them
        q = rnd(B, M, H, D, seed=seed, dtype=dtype).transpose(1, 2)
        k = rnd(B, N, H, D, seed=seed + 1, dtype=dtype).transpose(1, 2)
        v = rnd(B, N, H, D, seed=seed + 2, dtype=dtype).transpose(1, 2)
    else:
        q, k, v = (rnd(B, H, L, D, seed=seed + i, dtype=dtype) for i, L in enumerate((M, N, N)))
    table = rnd(nb, H, seed=seed + 3, scale=1.0) if bias else None
    out, lse = flash_attention_with_fusing_bias(q.to(dev), k.to(dev), v.to(dev), None if table is None else table.to(dev),
                                                causal=causal, sm_scale=sm_scale, NUM_BUCKETS=nb, MAX_DISTANCE=md,
                                                return_lse=True)
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == dtype
    want = O.dense_attention(q, k, v, table, causal, sm_scale, nb, md)
    err = (out.float().cpu() - want).abs().max().item()
    want_lse = O.dense_lse(q, k, table, causal, sm_scale, nb, md)
    fin = torch.isfinite(want_lse)
    lse_err = (lse.cpu()[fin] - want_lse[fin]).abs().max().item() if fin.any() else 0.0
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    return err, lse_err


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("M,N", [(128, 128), (256, 256), (100, 100), (1, 77), (77, 300), (300, 77), (513, 513)])
def test_dense_bf16_shapes(gpu_device, causal, M, N):
    err, lse_err = run_dense(gpu_device, 2, 3, M, N, 64, torch.bfloat16, causal)
    assert err <= TOL[torch.bfloat16], err
    assert lse_err <= 2e-2, lse_err


@pytest.mark.parametrize("D", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_dense_head_dims_and_dtypes(gpu_device, D, dtype):
    for causal in (False, True):
        err, lse_err = run_dense(gpu_device, 1, 2, 200, 200, D, dtype, causal, seed=5)
        assert err <= TOL[dtype], (err, causal)
        assert lse_err <= (1e-3 if dtype == torch.float32 else 2e-2)


def test_dense_strided_views(gpu_device):
    err, _ = run_dense(gpu_device, 2, 4, 333, 333, 64, torch.bfloat16, False, blhd=True, seed=7)
    assert err <= 2e-2
    err, _ = run_dense(gpu_device, 2, 4, 200, 200, 64, torch.float32, True, blhd=True, seed=8)
    assert err <= 1e-4


def test_dense_no_bias_default_scale(gpu_device):
    err, _ = run_dense(gpu_device, 1, 2, 150, 150, 64, torch.bfloat16, False, bias=False, sm_scale=None, seed=9)
    assert err <= 2e-2


def test_dense_other_bucket_params(gpu_device):
    for nb, md in ((64, 256), (16, 64), (32, 20)):
        err, _ = run_dense(gpu_device, 1, 2, 400, 400, 64, torch.float32, False, nb=nb, md=md, seed=10)
        assert err <= 1e-4, (nb, md, err)


def test_config2_shape_subset(gpu_device):
    """Baseline configuration 2 (B16 H12 L1024 D64 bf16, N(0,1)*0.5, table N(0,1)); oracle on 2 batches."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    g = torch.Generator().manual_seed(0)
    q, k, v = (0.5 * torch.randn(16, 12, 1024, 64, generator=g) for _ in range(3))
    table = torch.randn(32, 12, generator=g)
    qb, kb, vb = (t.to(torch.bfloat16) for t in (q, k, v))
    out = flash_attention_with_fusing_bias(qb.to(gpu_device), kb.to(gpu_device), vb.to(gpu_device),
                                           table.to(gpu_device), causal=False, sm_scale=1.0)
    for b in (0, 15):
        want = O.dense_attention(qb[b:b + 1], kb[b:b + 1], vb[b:b + 1], table, False, 1.0)
        assert (out[b:b + 1].float().cpu() - want).abs().max().item() <= 2e-2
    # literal bf16 'basic' (scores and weights rounded to bf16) is further from fp32 truth than the kernel
    lit = O.dense_attention(qb[:1], kb[:1], vb[:1], table, False, 1.0, compute_dtype=torch.bfloat16).float()
    assert (out[:1].float().cpu() - lit).abs().max().item() <= 4e-2


def test_long_sequence_properties(gpu_device):
    """L = 8192: V = 1 gives exactly 1; a constant table shift changes nothing (size-independent checks)."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    B, H, Lq, D = 1, 4, 8192, 64
    q = rnd(B, H, Lq, D, seed=11, dtype=torch.bfloat16).to(gpu_device)
    k = rnd(B, H, Lq, D, seed=12, dtype=torch.bfloat16).to(gpu_device)
    ones = torch.ones(B, H, Lq, D, dtype=torch.bfloat16, device=gpu_device)
    table = rnd(32, H, seed=13, scale=1.0).to(gpu_device)
    out = flash_attention_with_fusing_bias(q, k, ones, table, sm_scale=1.0)
    assert (out.float() - 1.0).abs().max().item() <= 1e-2
    v = rnd(B, H, Lq, D, seed=14, dtype=torch.bfloat16).to(gpu_device)
    a = flash_attention_with_fusing_bias(q, k, v, table, sm_scale=1.0)
    b = flash_attention_with_fusing_bias(q, k, v, table + 2.5, sm_scale=1.0)
    assert (a.float() - b.float()).abs().max().item() <= 1e-2
    # oracle on a random subset of 256 query rows of head 1
    rows = torch.randperm(Lq, generator=torch.Generator().manual_seed(15))[:256].sort().values
    qc, kc, vc = q.cpu()[:, 1:2], k.cpu()[:, 1:2], v.cpu()[:, 1:2]
    tb = table.cpu()[:, 1:2]
    i = rows[:, None]
    j = torch.arange(Lq)[None, :]
    bias = tb[O.relative_position_bucket(j - i, True, 32, 128)].permute(2, 0, 1).unsqueeze(0)
    want = O.basic_attention(qc[:, :, rows].float(), kc.float(), vc.float(), bias)
    assert (a[:, 1:2, rows].float().cpu() - want).abs().max().item() <= 2e-2


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_varlen(gpu_device, causal, dtype):
    from turbot5_amd.ops import flash_attention_with_fusing_bias_varlen
    H, D = 3, 64
    lens = [5, 128, 0, 129, 300, 1, 64]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    tot = int(cu[-1])
    q, k, v = (rnd(tot, H, D, seed=20 + i, dtype=dtype) for i in range(3))
    table = rnd(32, H, seed=23, scale=1.0)
    out, lse = flash_attention_with_fusing_bias_varlen(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                                       table.to(gpu_device), cu.to(gpu_device), cu.to(gpu_device),
                                                       max(lens), max(lens), causal=causal, sm_scale=1.0,
                                                       return_lse=True)
    want = O.varlen_attention(q, k, v, table, cu, cu, causal, 1.0)
    assert (out.float().cpu() - want).abs().max().item() <= TOL[dtype]
    assert lse.shape == (tot, H) and torch.isfinite(lse).all()


@pytest.mark.parametrize("causal", [False, True])
def test_padded_batch_in_place_with_seq_lens(gpu_device, causal):
    """Right-padded (B, L, H, D) batch viewed as (B*L, H, D): cu = b*L, lengths given separately.  Valid rows
    equal the packed oracle on the unpadded sequences; padding rows are never read (poisoned with NaN) and
    come back as zeros, like the reference's pad_input (padding.py:30-44)."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias_varlen
    B, L, H, D = 5, 200, 3, 64
    lens = [200, 1, 0, 129, 77]
    q, k, v = (rnd(B, L, H, D, seed=40 + i, dtype=torch.bfloat16) for i in range(3))
    table = rnd(32, H, seed=43, scale=1.0)
    for b, n in enumerate(lens):
        for t in (q, k, v):
            t[b, n:] = float("nan")
    cu_pad = torch.arange(0, (B + 1) * L, L, dtype=torch.int32)
    out, lse = flash_attention_with_fusing_bias_varlen(
        q.view(B * L, H, D).to(gpu_device), k.view(B * L, H, D).to(gpu_device), v.view(B * L, H, D).to(gpu_device),
        table.to(gpu_device), cu_pad.to(gpu_device), cu_pad.to(gpu_device), L, L, causal=causal, sm_scale=1.0,
        return_lse=True, seq_lens_q=torch.tensor(lens, dtype=torch.int32, device=gpu_device),
        seq_lens_k=torch.tensor(lens, dtype=torch.int32, device=gpu_device))
    out = out.float().cpu().view(B, L, H, D)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    packed = [torch.cat([t[b, :n] for b, n in enumerate(lens)]) for t in (q, k, v)]
    want = O.varlen_attention(*packed, table, cu, cu, causal, 1.0)
    for b, n in enumerate(lens):
        assert (out[b, :n] - want[cu[b]:cu[b + 1]]).abs().max().item() <= 2e-2 if n else True
        assert (out[b, n:] == 0).all()
    assert torch.isfinite(lse).all()


def test_varlen_cross_lengths(gpu_device):
    """different q and k lengths per sequence (decoder step over a padded cache)."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias_varlen
    H, D = 2, 64
    lq, lk = [1, 3, 130], [40, 200, 130]
    cq = torch.tensor([0] + list(np.cumsum(lq)), dtype=torch.int32)
    ck = torch.tensor([0] + list(np.cumsum(lk)), dtype=torch.int32)
    q = rnd(int(cq[-1]), H, D, seed=30, dtype=torch.bfloat16)
    k = rnd(int(ck[-1]), H, D, seed=31, dtype=torch.bfloat16)
    v = rnd(int(ck[-1]), H, D, seed=32, dtype=torch.bfloat16)
    table = rnd(32, H, seed=33, scale=1.0)
    for causal in (False, True):
        out = flash_attention_with_fusing_bias_varlen(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                                      table.to(gpu_device), cq.to(gpu_device), ck.to(gpu_device),
                                                      max(lq), max(lk), causal=causal, sm_scale=1.0)
        want = O.varlen_attention(q, k, v, table, cq, ck, causal, 1.0)
        assert (out.float().cpu() - want).abs().max().item() <= 2e-2


def test_dense_on_a_side_stream_and_under_graph_capture(gpu_device):
    """The library launches on the stream it is handed, allocates nothing and never synchronises: the op can
    run on a non-default stream and be captured into a device graph.  Every replay (with fresh inputs copied
    into the captured buffers, eager work and synchronisations in between) must equal the eager result."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    B, H, L, D = 2, 3, 384, 64
    table = rnd(32, H, seed=203, scale=1.0).to(gpu_device)
    sq, sk, sv = (torch.zeros(B, H, L, D, dtype=torch.bfloat16, device=gpu_device) for _ in range(3))
    side = torch.cuda.Stream(device=gpu_device)
    side.wait_stream(torch.cuda.current_stream(gpu_device))
    with torch.cuda.stream(side):
        for _ in range(3):                                   # warm-up outside the capture
            flash_attention_with_fusing_bias(sq, sk, sv, table, causal=True, sm_scale=1.0)
    torch.cuda.current_stream(gpu_device).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = flash_attention_with_fusing_bias(sq, sk, sv, table, causal=True, sm_scale=1.0)
    for rep in range(4):
        q, k, v = (rnd(B, H, L, D, seed=210 + 3 * rep + i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
        eager = flash_attention_with_fusing_bias(q, k, v, table, causal=True, sm_scale=1.0)
        torch.cuda.synchronize()
        sq.copy_(q); sk.copy_(k); sv.copy_(v)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), f"replay {rep} differs from the eager launch"
    want = O.dense_attention(q.cpu(), k.cpu(), v.cpu(), table.cpu(), True, 1.0)
    assert (captured.float().cpu() - want).abs().max().item() <= 2e-2


@pytest.mark.parametrize("B,H,M,N", [(1, 12, 2048, 2048), (3, 5, 700, 700), (1, 1, 1500, 1500), (2, 3, 384, 1000),
                                     (5, 7, 129, 129), (1, 12, 3000, 3000), (16, 12, 1024, 1024), (2, 3, 1000, 384)])
def test_causal_item_order_writes_every_row(gpu_device, B, H, M, N):
    """The causal launch cuts the item list into per-XCD slices of equal work and walks each slice longest
    tile first; every (batch, head, tile) must still be computed exactly once.  Output and lse start as NaN
    so that a tile nobody computed cannot pass by luck."""
    import ctypes as C
    from turbot5_amd import _lib as L
    from turbot5_amd import ops
    dt = torch.bfloat16
    q, k, v = (rnd(B, H, n, 64, seed=40 + i, dtype=dt).to(gpu_device) for i, n in enumerate((M, N, N)))
    table = rnd(32, H, seed=43, scale=1.0).to(gpu_device)
    o = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, M), float("nan"), device=gpu_device, dtype=torch.float32)
    a = L.T5ADenseArgs()
    a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr()
    a.q_strides, a.k_strides, a.v_strides, a.o_strides = (ops._strides3(t) for t in (q, k, v, o))
    a.dtype, a.B, a.H, a.M, a.N, a.D = L.T5A_BF16, B, H, M, N, 64
    a.causal, a.sm_scale = 1, 1.0
    a.bias, keep = ops._bias_struct(table, H, 32, 128, q)
    L.check(L.load().t5a_fwd_dense(C.byref(a), ops._stream(q)))
    torch.cuda.synchronize()
    want = O.dense_attention(q.cpu(), k.cpu(), v.cpu(), table.cpu(), True, 1.0)
    want_lse = O.dense_lse(q.cpu(), k.cpu(), table.cpu(), True, 1.0)
    got = o.float().cpu()
    assert not torch.isnan(got).any(), "rows left unwritten"
    assert (got - want).abs().max().item() <= TOL[dt]
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max().item() <= 2e-2


def _plan_case(name):
    g = torch.Generator().manual_seed(11)
    if name == "mixed":            # lengths as a tokenised batch has them, one empty sequence
        lq = torch.randint(1, 1500, (40,), generator=g).tolist()
        lq[7] = 0
        return lq, lq
    if name == "spill":            # a few long and many short sequences: the XCDs that take the short ones
        lq = [4000] * 3 + [100] * 300   # hold far more items than their share of slots
        return lq, lq
    if name == "cross":            # keys longer than queries (cache), and shorter
        lq = torch.randint(1, 1100, (64,), generator=g).tolist()
        lk = [max(1, n + int(d)) for n, d in zip(lq, torch.randint(-300, 600, (64,), generator=g).tolist())]
        return lq, lk
    raise KeyError(name)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", ["mixed", "spill", "cross"])
def test_varlen_launch_plan(gpu_device, case, causal):
    """Larger packed launches run from a device-built plan (per-XCD item lists of equal work).  The plan only
    reorders items: the result equals, bit for bit, the one of the launch that walks cu_seqlens, and both
    match the oracle.  The planned launch runs first, so memory left by the other cannot stand in for it."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias_varlen
    H, D = 4, 64
    lq, lk = _plan_case(case)
    cq = torch.tensor([0] + list(np.cumsum(lq)), dtype=torch.int32)
    ck = torch.tensor([0] + list(np.cumsum(lk)), dtype=torch.int32)
    q = rnd(int(cq[-1]), H, D, seed=50, dtype=torch.bfloat16)
    k = rnd(int(ck[-1]), H, D, seed=51, dtype=torch.bfloat16)
    v = rnd(int(ck[-1]), H, D, seed=52, dtype=torch.bfloat16)
    table = rnd(32, H, seed=53, scale=1.0)
    dev = [t.to(gpu_device) for t in (q, k, v, table, cq, ck)]
    outs = []
    for plan in ("always", False):
        o, lse = flash_attention_with_fusing_bias_varlen(*dev, max(lq), max(lk), causal=causal, sm_scale=1.0,
                                                         return_lse=True, launch_plan=plan)
        torch.cuda.synchronize()
        outs.append((o.cpu(), lse.cpu()))
    assert torch.equal(outs[0][0].view(torch.int16), outs[1][0].view(torch.int16))
    assert torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32))
    want = O.varlen_attention(q, k, v, table, cq, ck, causal, 1.0)
    assert (outs[0][0].float() - want).abs().max().item() <= 2e-2


def test_varlen_launch_plan_with_padding_rows(gpu_device):
    """planned launch over a right-padded batch given as cu = b * L plus lengths"""
    from turbot5_amd.ops import flash_attention_with_fusing_bias_varlen
    B, Lp, H, D = 24, 1024, 6, 64
    lens = torch.randint(0, Lp + 1, (B,), generator=torch.Generator().manual_seed(12)).tolist()
    lens[3] = Lp
    q, k, v = (rnd(B * Lp, H, D, seed=60 + i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
    table = rnd(32, H, seed=63, scale=1.0).to(gpu_device)
    cu = torch.arange(0, (B + 1) * Lp, Lp, dtype=torch.int32, device=gpu_device)
    ln = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
    outs = [flash_attention_with_fusing_bias_varlen(q, k, v, table, cu, cu, Lp, Lp, causal=False, sm_scale=1.0,
                                                    seq_lens_q=ln, seq_lens_k=ln, launch_plan=plan).cpu()
            for plan in ("always", False)]
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    o = outs[0].view(B, Lp, H, D)
    for b, n in enumerate(lens):
        assert (o[b, n:] == 0).all()
    b = 3
    want = O.dense_attention(*(t.view(B, Lp, H, D)[b:b + 1].transpose(1, 2).cpu() for t in (q, k, v)), table.cpu(), False, 1.0)
    assert (o[b:b + 1].transpose(1, 2).float() - want).abs().max().item() <= 2e-2


def test_launch_plan_object_is_reused_and_rebuilt(gpu_device):
    """One LaunchPlan over several calls: built by the first, found ready by the next (other q/k/v, same
    lengths), rebuilt when the lengths are another tensor.  Every result equals the unplanned launch."""
    from turbot5_amd.ops import LaunchPlan, flash_attention_with_fusing_bias_varlen
    H, D = 4, 64
    table = rnd(32, H, seed=73, scale=1.0).to(gpu_device)
    plan = LaunchPlan()
    g = torch.Generator().manual_seed(13)
    built = []
    for step, seed in enumerate((70, 71, 72)):
        if step != 1:   # step 1 keeps the tensors of step 0
            lens = torch.randint(600, 1400, (48,), generator=g).tolist()   # enough tiles for a plan
            cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=gpu_device)
        q, k, v = (rnd(int(cu[-1]), H, D, seed=seed + 10 * i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
        key_before = plan.key
        got = flash_attention_with_fusing_bias_varlen(q, k, v, table, cu, cu, max(lens), max(lens), causal=True,
                                                      sm_scale=1.0, launch_plan=plan)
        built.append(plan.key != key_before)
        want = flash_attention_with_fusing_bias_varlen(q, k, v, table, cu, cu, max(lens), max(lens), causal=True,
                                                       sm_scale=1.0, launch_plan=False)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), step
    assert built == [True, False, True]


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("lens", [[5, 128, 0, 129, 300, 1, 64], [700], [0, 0, 3], [129] * 9, [1] * 40])
def test_launch_plan_of_tiny_batches(gpu_device, lens, causal):
    """plans of a handful of items: empty sequences, one sequence, fewer items than XCDs"""
    from turbot5_amd.ops import flash_attention_with_fusing_bias_varlen
    H, D = 3, 64
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    q, k, v = (rnd(int(cu[-1]), H, D, seed=80 + i, dtype=torch.bfloat16) for i in range(3))
    table = rnd(32, H, seed=83, scale=1.0)
    out = flash_attention_with_fusing_bias_varlen(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                                  table.to(gpu_device), cu.to(gpu_device), cu.to(gpu_device),
                                                  max(lens), max(lens), causal=causal, sm_scale=1.0,
                                                  launch_plan="always")
    want = O.varlen_attention(q, k, v, table, cu, cu, causal, 1.0)
    assert (out.float().cpu() - want).abs().max().item() <= 2e-2


@pytest.mark.parametrize("causal", [False, True])
def test_bias_lut_buffer_gives_identical_results(gpu_device, causal):
    """The LUTs of all heads, built once into a buffer and fetched by later launches, are the image a work item
    otherwise builds for itself: outputs are bit-identical with and without the buffer, on the launch that
    builds it and on the ones that find it ready; an in-place update of the table makes a new buffer."""
    from turbot5_amd import ops
    B, H, M, D = 2, 5, 700, 64
    q, k, v = (rnd(B, H, M, D, seed=90 + i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
    table = rnd(32, H, seed=93, scale=1.0).to(gpu_device)
    run = lambda: ops.flash_attention_with_fusing_bias(q, k, v, table, causal=causal, sm_scale=1.0).cpu()  # noqa: E731
    ops._BIAS_LUTS.clear()
    ops.BIAS_LUT_CACHE = False
    try:
        plain = run()
    finally:
        ops.BIAS_LUT_CACHE = True
    assert len(ops._BIAS_LUTS) == 0
    first, second = run(), run()
    assert len(ops._BIAS_LUTS) == 1
    assert torch.equal(plain.view(torch.int16), first.view(torch.int16))
    assert torch.equal(plain.view(torch.int16), second.view(torch.int16))
    table.mul_(-0.5)   # same storage, new values
    third = run()
    assert len(ops._BIAS_LUTS) == 2
    want = O.dense_attention(q.cpu(), k.cpu(), v.cpu(), table.cpu(), causal, 1.0)
    assert (third.float() - want).abs().max().item() <= TOL[torch.bfloat16]
    assert not torch.equal(third.view(torch.int16), plain.view(torch.int16))


@pytest.mark.parametrize("tdtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("layout", ["plain", "offset", "transposed"])
def test_bias_table_dtypes_and_layouts(gpu_device, tdtype, layout):
    """The kernel reads the (NUM_BUCKETS, H) table in its own type and strides: 16-bit tables, a table that
    starts in the middle of a 4-byte word, and the transposed (H, NUM_BUCKETS) storage, with and without
    the LUT buffer."""
    from turbot5_amd import ops
    B, H, M, D = 1, 3, 300, 64
    q, k, v = (rnd(B, H, M, D, seed=100 + i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
    vals = rnd(32, H, seed=103, scale=1.0).to(tdtype)
    if layout == "plain":
        table = vals.to(gpu_device)
    elif layout == "offset":
        buf = torch.zeros(32 * H + 1, dtype=tdtype, device=gpu_device)
        buf[1:] = vals.reshape(-1).to(gpu_device)
        table = buf[1:].view(32, H)
    else:
        table = vals.t().contiguous().to(gpu_device).t()
    assert table.shape == (32, H)
    want = O.dense_attention(q.cpu(), k.cpu(), v.cpu(), vals.float(), False, 1.0)
    for cache in (False, True):
        ops.BIAS_LUT_CACHE = cache
        try:
            got = ops.flash_attention_with_fusing_bias(q, k, v, table, causal=False, sm_scale=1.0)
        finally:
            ops.BIAS_LUT_CACHE = True
        assert (got.float().cpu() - want).abs().max().item() <= TOL[torch.bfloat16], (cache, layout, tdtype)


def test_packed_batch_with_a_shared_plan_under_graph_capture(gpu_device):
    """A packed launch with a launch plan inside a device graph: the plan is rebuilt inside the graph (a plan
    recorded during capture has not run, and one built before may be overwritten before a replay), so replays
    follow the lengths that the captured cu_seqlens buffer holds at that moment.  The LaunchPlan object given
    to the captured call is left untouched and still serves eager calls."""
    from turbot5_amd.ops import LaunchPlan, flash_attention_with_fusing_bias_varlen
    H, D, total = 4, 64, 30000
    table = rnd(32, H, seed=303, scale=1.0).to(gpu_device)
    sq, sk, sv = (torch.zeros(total, H, D, dtype=torch.bfloat16, device=gpu_device) for _ in range(3))
    cu = torch.zeros(41, dtype=torch.int32, device=gpu_device)

    def lengths(seed):
        g = torch.Generator().manual_seed(seed)
        cut = torch.sort(torch.randperm(total - 1, generator=g)[:39] + 1).values
        return torch.cat([torch.tensor([0]), cut, torch.tensor([total])]).to(torch.int32)

    cu.copy_(lengths(1))
    plan = LaunchPlan()
    call = lambda: flash_attention_with_fusing_bias_varlen(sq, sk, sv, table, cu, cu, total, total, causal=False,  # noqa: E731
                                                           sm_scale=1.0, launch_plan=plan)
    for _ in range(2):
        call()                                               # builds the shared plan eagerly
    torch.cuda.synchronize()
    key = plan.key
    assert key is not None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = call()
    assert plan.key == key                                   # the capture did not touch the shared plan
    for rep in range(3):
        q, k, v = (rnd(total, H, D, seed=310 + 3 * rep + i, dtype=torch.bfloat16).to(gpu_device) for i in range(3))
        new_cu = lengths(2 + rep).to(gpu_device)
        eager = flash_attention_with_fusing_bias_varlen(q, k, v, table, new_cu, new_cu, total, total, causal=False,
                                                        sm_scale=1.0, launch_plan=False)
        torch.cuda.synchronize()
        sq.copy_(q); sk.copy_(k); sv.copy_(v); cu.copy_(new_cu)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), f"replay {rep} differs from the eager launch"


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_scores_that_keep_climbing_along_the_keys(gpu_device, dtype, causal):
    """The running row maximum has to be raised again and again: scores grow by 16 powers of two per
    64 keys.  sm_scale = ln 2 makes the kernel's base-2 scaling of Q an identity and the ramp is a
    small integer, so the scores themselves are exact and the usual tolerance applies."""
    import math
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    B, H, L, D = 1, 2, 1500, 64
    q, k, v = (rnd(B, H, L, D, seed=40 + i, dtype=dtype) for i in range(3))
    q[..., 0] = 2.0
    k[..., 0] = (torch.arange(L) // 16 * 2).to(dtype)
    table = rnd(32, H, seed=43, scale=1.0)
    sm = math.log(2.0)
    out, lse = flash_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), table.to(gpu_device),
                                                causal=causal, sm_scale=sm, return_lse=True)
    want = O.dense_attention(q, k, v, table, causal, sm)
    want_lse = O.dense_lse(q, k, table, causal, sm)
    tol = 5e-4 if dtype == torch.float32 else TOL[dtype]     # fp32: scores reach 250, one rounding of the scale shows
    assert (out.float().cpu() - want).abs().max().item() <= tol
    # the row sum adds probabilities as the matrix core sees them (rounded to the 16-bit type)
    assert (lse.cpu() - want_lse).abs().max().item() <= (2e-3 if dtype == torch.float32 else 1e-2)


def test_raw_ctypes_binding_as_a_reference_maintainer_would_write_it(gpu_device):
    """The binding shown to maintainers of the reference (a drop-in body for flash_attn_v2_fwd_bias,
    fused_bias_attention.py:23-59): plain ctypes on the C ABI, no helper of the ops module."""
    import ctypes as C
    from turbot5_amd._lib import load, check, T5ADenseArgs, T5A_BF16

    def flash_attn_v2_fwd_bias(q, k, v, bias_weights, causal, sm_scale):
        B, H, M, D = q.shape
        o = torch.empty_like(q)
        lse = torch.empty((B, H, M), device=q.device, dtype=torch.float32)
        a = T5ADenseArgs()
        a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr()
        for name, t in (("q_strides", q), ("k_strides", k), ("v_strides", v), ("o_strides", o)):
            setattr(a, name, (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2)))
        a.dtype, a.B, a.H, a.M, a.N, a.D = T5A_BF16, B, H, M, k.shape[2], D
        a.causal, a.sm_scale = int(causal), float(sm_scale)
        if bias_weights is not None:
            a.bias.table, a.bias.table_dtype = bias_weights.data_ptr(), 1
            a.bias.num_buckets, a.bias.max_distance = 32, 128
            a.bias.stride_bucket, a.bias.stride_head = bias_weights.stride(0), bias_weights.stride(1)
        with torch.cuda.device(q.device):
            check(load().t5a_fwd_dense(C.byref(a), torch.cuda.current_stream().cuda_stream))
        return o, lse

    q, k, v = (rnd(2, 4, 300, 64, seed=70 + i, dtype=torch.bfloat16) for i in range(3))
    table = rnd(32, 4, seed=73, scale=1.0)
    for causal in (False, True):
        o, lse = flash_attn_v2_fwd_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), table.to(gpu_device), causal, 1.0)
        want = O.dense_attention(q, k, v, table, causal, 1.0)
        assert (o.float().cpu() - want).abs().max().item() <= TOL[torch.bfloat16]
        assert (lse.cpu() - O.dense_lse(q, k, table, causal, 1.0)).abs().max().item() <= 2e-2


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D", [16, 32, 64, 128])
def test_output_in_token_major_layout_with_guard_rows(gpu_device, dt, D):
    """The write-back stores rows in 16-byte pieces (after an exchange between the halves of a wavefront): output in
    (B, M, H, D) layout through the C ABI, a ragged number of rows, every head dimension; rows and heads that do not
    belong to the call keep their fill value."""
    import ctypes as C
    from turbot5_amd import _lib as L
    from turbot5_amd import ops
    B, H, M, N = 2, 3, 77, 150
    q, k, v = (rnd(B, H, n, D, seed=300 + i, dtype=dt).to(gpu_device) for i, n in enumerate((M, N, N)))
    table = rnd(32, H, seed=303, scale=1.0).to(gpu_device)
    fill = 123.0
    buf = torch.full((B, M + 3, H + 1, D), fill, device=gpu_device, dtype=dt)      # guard rows and a guard head
    o = buf[:, :M, :H].permute(0, 2, 1, 3)                                          # (B, H, M, D) view, rows H + 1 heads apart
    a = L.T5ADenseArgs()
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    a.q_strides, a.k_strides, a.v_strides, a.o_strides = (ops._strides3(t) for t in (q, k, v, o))
    a.dtype = {torch.bfloat16: L.T5A_BF16, torch.float16: L.T5A_F16, torch.float32: L.T5A_F32}[dt]
    a.B, a.H, a.M, a.N, a.D = B, H, M, N, D
    a.causal, a.sm_scale = 0, 1.0
    a.bias, keep = ops._bias_struct(table, H, 32, 128, q)
    L.check(L.load().t5a_fwd_dense(C.byref(a), ops._stream(q)))
    torch.cuda.synchronize()
    want = O.dense_attention(q.cpu(), k.cpu(), v.cpu(), table.cpu(), False, 1.0)
    got = o.float().cpu()
    assert (got - want).abs().max().item() <= TOL[dt]
    host = buf.float().cpu()
    assert (host[:, M:] == fill).all() and (host[:, :, H] == fill).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("kind", ["ramp", "late_outlier", "early_outlier", "huge_everywhere", "tiny_everywhere"])
def test_running_max_is_raised_from_the_row_sums(gpu_device, dtype, causal, kind):
    """The dense fast steps at head_dim 64 form no row maximum: a tile's row sum tells whether the running max must
    be raised, and a rare block then looks the exact maximum up and forms the tile's exponentials again, before the
    tile reaches the output accumulators.  Scores built to exercise that block:
      ramp             every key tile scores about 40 above the one before it (base-2 units): a raise in every step
      late_outlier     one key near the end scores 300 above everything: its exponential overflows fp32 against the
                       stale maximum, and must never reach the accumulators
      early_outlier    the same in the first tile: everything later underflows against it
      huge / tiny      all scores around +400 / -400: no probability may overflow or underflow as a whole
    Keys are multiples of one direction u, queries carry a unit component along u, so q.k is the key's multiple and
    exact in the 16-bit types; values are random.  Against the oracle in fp32 on the same inputs."""
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    B, H, L, D = 1, 2, 1024, 64
    g = torch.Generator().manual_seed(77)
    u = torch.zeros(D)
    u[0] = 1.0
    q = 0.05 * torch.randn(B, H, L, D, generator=g)
    q[..., 0] = 1.0                                     # q . (c u) = c
    j = torch.arange(L, dtype=torch.float32)
    if kind == "ramp":
        c = 28.0 * (j // 64)                            # nats: about 40 per tile in base-2 units
    elif kind == "late_outlier":
        c = torch.zeros(L)
        c[L - 37] = 208.0
    elif kind == "early_outlier":
        c = torch.zeros(L)
        c[5] = 208.0
    elif kind == "huge_everywhere":
        c = 280.0 + (j % 7)
    else:
        c = -280.0 - (j % 7)
    if dtype == torch.float16:
        c = c * 0.5                                     # (fp16 holds the keys' multiples up to 65504; keep them exact)
    k = (c[:, None] * u[None, :]).expand(B, H, L, D).clone()
    k[..., 1:] = 0.05 * torch.randn(B, H, L, D - 1, generator=g)
    v = torch.randn(B, H, L, D, generator=g)
    q, k, v = (t.to(dtype) for t in (q, k, v))
    table = torch.randn(32, H, generator=g)
    want = O.dense_attention(q, k, v, table, causal, 1.0)
    for exact in (None, True):
        got = flash_attention_with_fusing_bias(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), table.to(gpu_device),
                                               causal=causal, sm_scale=1.0, exact_scores=exact).float().cpu()
        assert torch.isfinite(got).all(), (kind, exact)
        # (scores this large make one key's weight 1: the default mode's extra rounding of Q moves scores of several
        # hundred by whole units, so it is compared on the kinds whose result does not hang on a single unit)
        if exact or kind in ("late_outlier", "early_outlier"):
            assert (got - want).abs().max().item() <= 3e-2, (kind, exact)
