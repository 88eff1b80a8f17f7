"""Function-level API of the attention hot path, with the reference's signatures.

``flash_attention_with_fusing_bias`` and ``flash_attention_with_fusing_bias_varlen``
keep the names, argument order and defaults of the reference
(src/turbot5/ops/fused_bias_attention.py:876-890, varlen_fused_bias_attn.py:870-889);
``flash_attn_v2_fwd`` keeps those of src/turbot5/ops/flash_decoding.py:6.
All of them launch hand-written HIP kernels through libt5attn.so; tensors must
live on a ROCm device.  Forward only: the outputs carry no autograd graph.
"""
from __future__ import annotations

import ctypes as C
import math
from collections import OrderedDict
from typing import Optional, Tuple

import torch

from . import _lib as L

_DTYPES = {torch.bfloat16: L.T5A_BF16, torch.float32: L.T5A_F32, torch.float16: L.T5A_F16}

# Score precision of the fused kernels for bf16 / fp16 inputs when a call does not say (``exact_scores=None``).
# False: the query rows are multiplied by sm_scale * log2(e) and rounded back to the input type before the
# matrix product (relative error 2^-9 per term in bf16; still 3.6 times more accurate than the reference's
# 'basic' path in bf16, and within 2e-2 of fp32 math for scores of deviation up to about 4).  True: the factor
# is applied to the fp32 product, as the reference's fused kernel does (one more multiply per score).
# "prescaled" (per call only): q already carries sm_scale * log2(e), see ``prescaled_query``; the kernel applies
# no factor, so q was rounded to its type once -- the accuracy of True at the speed of False.
EXACT_SCORES = False
LOG2E = 1.4426950408889634

# Sparse patterns: q tiles per work item (0: the library chooses from the shape and the device).  Results do not
# depend on it; tests pin every path of the run logic with it.
RUN_LEN = 0

# Backward of 16-bit tensors at head_dim 64.  False: the 16-bit matrix cores, probabilities and dS rounded to the
# tensors' type before the products that form dq, dk and dv, as the reference's kernels round them
# (fused_bias_attention.py:575-590).  True: every product on the fp32 matrix cores (about five times slower).
BACKWARD_FP32_MATH = False


def _exact(flag) -> int:
    if isinstance(flag, str):
        if flag != "prescaled":
            raise ValueError(f"exact_scores={flag!r}: None, False, True or 'prescaled'")
        return L.SCORES_PRESCALED
    return int(EXACT_SCORES if flag is None else bool(flag))


def prescaled_query(hidden: torch.Tensor, weight: torch.Tensor, dtype: torch.dtype, sm_scale: float = 1.0) -> torch.Tensor:
    """The query projection with sm_scale * log2(e) folded in: ``hidden @ weight.T * (sm_scale * log2 e)`` rounded to
    ``dtype`` ONCE, for ``exact_scores="prescaled"``.  Activations that are already in ``dtype`` take the factor
    as the GEMM's alpha (applied to the fp32 accumulator, before the rounding of the output); wider activations
    are multiplied on their way into the cast."""
    c = float(sm_scale) * LOG2E
    x2 = hidden.reshape(-1, hidden.shape[-1])
    if x2.dtype == dtype and weight.dtype == dtype:
        q = torch.addmm(x2.new_zeros(1), x2, weight.t(), beta=0, alpha=c)
    else:
        q = torch.mul(torch.nn.functional.linear(x2, weight), c).to(dtype)
    return q.view(*hidden.shape[:-1], weight.shape[0])


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected bfloat16, float16 or float32") from None


def _check_inputs(q, k, v):
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("q, k, v must be on a ROCm device: this path has no CPU implementation")
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError(f"q, k, v dtypes differ: {q.dtype}, {k.dtype}, {v.dtype}")
    Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Dq == Dk == Dv                       # fused_bias_attention.py:827
    assert Dk in {16, 32, 64, 128}              # fused_bias_attention.py:828


def _forward_only(what: str, *tensors):
    """The sparse patterns, split-K decoding and the RMS norm kernel have no backward: say so instead of returning
    a result that silently carries no graph."""
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise NotImplementedError(f"{what} is forward only (no backward kernel); run it under torch.no_grad() or "
                                  "use attention_type='flash', whose kernels have one")


def _unit(t: torch.Tensor) -> int:
    return 4 if t.dtype == torch.float32 else 8


def _kernel_ready(t: torch.Tensor) -> torch.Tensor:
    """The kernels need head_dim contiguous, 16-byte aligned rows; copy only when that fails."""
    u = _unit(t)
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % u == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


# Distance LUTs of the bias tables seen lately, built on the device by the first launch that uses a table and
# fetched by the later ones.  Keyed by the table's identity and version (so an optimiser step or any other
# in-place update makes a new entry), the bucket parameters and the stream the build was queued on; the entry
# keeps the table alive, so its address cannot be taken by another tensor.
_BIAS_LUTS: "OrderedDict[tuple, tuple]" = OrderedDict()
BIAS_LUT_CACHE = True


def _bias_lut(b, bias: torch.Tensor, H: int, num_buckets: int, max_distance: int, causal: bool, ref: torch.Tensor,
              window: int = 0):
    """-> (lut buffer or None, cache key to commit after a successful launch or None).
    window > 0: the images with that sliding window folded in (what the local pattern's work items fetch)."""
    if not BIAS_LUT_CACHE or torch.cuda.is_current_stream_capturing():
        return None, None   # a build recorded into a graph would not have run when the next eager launch reads it
    key = (bias.data_ptr(), bias._version, bias.stride(0), bias.stride(1), bias.dtype, H, num_buckets, max_distance,
           bool(causal), ref.device.index, _stream(ref), int(window))
    hit = _BIAS_LUTS.get(key)
    pending = None
    if hit is None:
        nbytes = (L.load().t5a_bias_lut_bytes_windowed(H, num_buckets, max_distance, int(window)) if window > 0
                  else L.load().t5a_bias_lut_bytes(H, num_buckets, max_distance, int(bool(causal))))
        if nbytes <= 0:
            return None, None
        lut = torch.empty(nbytes, device=ref.device, dtype=torch.uint8)
        pending = key       # recorded as built only once the library has queued the build (_commit_lut)
        b.lut_ready = 0
    else:
        lut = hit[1]
        b.lut_ready = 1
    b.lut, b.lut_bytes, b.lut_window = lut.data_ptr(), lut.numel(), int(window)
    return lut, pending


def _commit_lut(keep, launched: bool):
    """After the library call has returned without error: remember a LUT buffer that this call built.  A call
    that returned before its launch (empty batch) or raised has not built it, and leaves no entry."""
    if keep is None or not launched:
        return
    table, lut, pending, bias = keep
    if pending is not None and lut is not None:
        _BIAS_LUTS[pending] = (bias, lut)
        while len(_BIAS_LUTS) > 64:
            _BIAS_LUTS.popitem(last=False)


def clear_bias_luts():
    """Forget every cached distance LUT.  The cache keys on the table's identity and version counter; updates
    that bypass the counter (``param.data.copy_``, raw kernels writing into the table) need this call."""
    _BIAS_LUTS.clear()


def _bias_struct(bias: Optional[torch.Tensor], H: int, num_buckets: int, max_distance: int, ref: torch.Tensor,
                 causal: bool = False, window: int = 0):
    b = L.T5ABias()
    if bias is None:
        b.table = None
        return b, None
    if bias.dim() != 2 or bias.shape[0] != num_buckets or bias.shape[1] != H:
        raise ValueError(f"bias table must be (NUM_BUCKETS={num_buckets}, H={H}), got {tuple(bias.shape)}")
    if bias.device != ref.device:
        raise RuntimeError("bias table must be on the same device as q")
    table = bias.detach()
    if table.dtype not in _DTYPES:
        table = table.float()
    b.table = table.data_ptr()
    b.table_dtype = _DTYPES[table.dtype]
    b.num_buckets = num_buckets
    b.max_distance = max_distance
    b.stride_bucket = table.stride(0)
    b.stride_head = table.stride(1)
    lut, pending = (_bias_lut(b, bias, H, num_buckets, max_distance, causal, ref, window)
                    if table.data_ptr() == bias.data_ptr() else (None, None))
    return b, (table, lut, pending, bias)   # alive until the launch has been queued; see _commit_lut


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """hipStream_t of torch's current stream on t's device (the raw getter skips a Stream object per call)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _on_device:
    """Makes t's device current for the launch; a no-op (no context switch) when it already is."""

    def __init__(self, t: torch.Tensor):
        idx = t.device.index
        self.ctx = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)


def _strides3(t):
    return (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def _dense_forward(q, k, v, bias, causal, sm_scale, NUM_BUCKETS, MAX_DISTANCE, return_lse, exact_scores):
    _check_inputs(q, k, v)
    B, H, M, D = q.shape
    N = k.shape[2]
    if k.shape[0] != B or k.shape[1] != H or v.shape != k.shape:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    q_, k_, v_ = (_kernel_ready(t) for t in (q, k, v))
    o = torch.empty_like(q_)
    lse = torch.empty((B, H, M), device=q.device, dtype=torch.float32) if return_lse else None
    a = L.T5ADenseArgs()
    a.q, a.k, a.v, a.o = q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr()
    a.lse = lse.data_ptr() if lse is not None else None
    a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides3(q_), _strides3(k_), _strides3(v_), _strides3(o)
    a.dtype, a.B, a.H, a.M, a.N, a.D = _dtype_code(q), B, H, M, N, D
    a.causal, a.sm_scale = int(bool(causal)), float(sm_scale)
    a.exact_scores = _exact(exact_scores)
    a.bias, keep = _bias_struct(bias, H, NUM_BUCKETS, MAX_DISTANCE, q, causal)
    with _on_device(q):
        L.check(L.load().t5a_fwd_dense(C.byref(a), _stream(q)))
    _commit_lut(keep, B > 0 and M > 0)
    return (o, lse) if return_lse else o


def _dense_backward(q, k, v, bias, o, lse, dout, causal, sm_scale, NUM_BUCKETS, MAX_DISTANCE, exact_scores):
    """-> dq, dk, dv, dbias (fp32 (NUM_BUCKETS, H), or None without a table); t5a_bwd_dense"""
    B, H, M, D = q.shape
    N = k.shape[2]
    if D == 128 and (q.dtype == torch.float32 or BACKWARD_FP32_MATH):
        raise NotImplementedError("backward at head_dim 128: bf16 / fp16 tensors only (the fp32 kernels cover head_dim 16, 32 and 64)")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    q_, k_, v_, o_, g_ = (_kernel_ready(t) for t in (q, k, v, o, dout))
    dq, dk, dv = torch.empty_like(q_), torch.empty_like(k_), torch.empty_like(v_)
    dtable = torch.empty((NUM_BUCKETS, H), device=q.device, dtype=torch.float32) if bias is not None else None
    lib = L.load()
    ws = torch.empty(max(int(lib.t5a_bwd_workspace_bytes(B, H, M)), 16), device=q.device, dtype=torch.uint8)
    a = L.T5ADenseBwdArgs()
    a.q, a.k, a.v, a.o, a.dout, a.lse = (t.data_ptr() for t in (q_, k_, v_, o_, g_, lse))
    a.dq, a.dk, a.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    a.dtable = dtable.data_ptr() if dtable is not None else None
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    for name, t in (("q_strides", q_), ("k_strides", k_), ("v_strides", v_), ("o_strides", o_), ("dout_strides", g_),
                    ("dq_strides", dq), ("dk_strides", dk), ("dv_strides", dv)):
        setattr(a, name, _strides3(t))
    a.dtype, a.B, a.H, a.M, a.N, a.D = _dtype_code(q), B, H, M, N, D
    a.causal, a.sm_scale = int(bool(causal)), float(sm_scale)
    a.exact_scores = _exact(exact_scores)
    a.fp32_math = int(bool(BACKWARD_FP32_MATH))
    b = L.T5ABias()
    keep = None
    if bias is not None:
        table = bias.detach()
        if table.dtype not in _DTYPES:
            table = table.float()
        b.table, b.table_dtype = table.data_ptr(), _DTYPES[table.dtype]
        b.num_buckets, b.max_distance = NUM_BUCKETS, MAX_DISTANCE
        b.stride_bucket, b.stride_head = table.stride(0), table.stride(1)
        keep = table
    a.bias = b
    with _on_device(q):
        L.check(lib.t5a_bwd_dense(C.byref(a), _stream(q)))
    del keep
    return dq, dk, dv, dtable


class FlashAttentionBias(torch.autograd.Function):
    """The dense fused-bias forward with its backward (reference fused_bias_attention.py:821-873): gradients for q,
    k, v and the (NUM_BUCKETS, H) table."""

    @staticmethod
    def forward(ctx, q, k, v, bias, causal, sm_scale, NUM_BUCKETS, MAX_DISTANCE, exact_scores):
        o, lse = _dense_forward(q, k, v, bias, causal, sm_scale, NUM_BUCKETS, MAX_DISTANCE, True, exact_scores)
        ctx.save_for_backward(q, k, v, o, lse, *(() if bias is None else (bias,)))
        ctx.has_bias = bias is not None
        ctx.args = (bool(causal), sm_scale, NUM_BUCKETS, MAX_DISTANCE, exact_scores)
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, dout, _dlse):
        q, k, v, o, lse = ctx.saved_tensors[:5]
        bias = ctx.saved_tensors[5] if ctx.has_bias else None
        causal, sm_scale, nb, md, exact = ctx.args
        dq, dk, dv, dtable = _dense_backward(q, k, v, bias, o, lse, dout, causal, sm_scale, nb, md, exact)
        dbias = dtable.to(bias.dtype) if bias is not None and ctx.needs_input_grad[3] else None
        return dq, dk, dv, dbias, None, None, None, None, None


def flash_attention_with_fusing_bias(q, k, v, bias, causal=False, sm_scale=None, NUM_BUCKETS=32, MAX_DISTANCE=128,
                                     return_lse: bool = False, exact_scores: Optional[bool] = None):
    """FlashAttention forward with the T5 relative-position bias computed inside the kernel.

    q (B,H,M,D); k, v (B,H,N,D), any batch/head/row strides; ``bias`` is the
    (NUM_BUCKETS, H) table or None.  ``causal`` selects the causal mask and the
    unidirectional buckets together.  ``sm_scale=None`` means 1/sqrt(D).  Returns
    a tensor shaped and strided like q (``empty_like``), plus the (B,H,M) fp32
    log-sum-exp when ``return_lse``.  Differentiable in q, k, v and the table (fp32 tensors: head_dim up to 64), as the
    reference's autograd function is (fused_bias_attention.py:821-873).
    """
    needs_grad = torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (q, k, v, bias))
    if needs_grad:
        o, lse = FlashAttentionBias.apply(q, k, v, bias, causal, sm_scale, NUM_BUCKETS, MAX_DISTANCE, exact_scores)
        return (o, lse) if return_lse else o
    return _dense_forward(q, k, v, bias, causal, sm_scale, NUM_BUCKETS, MAX_DISTANCE, return_lse, exact_scores)


PLAN_MIN_ITEMS = 3072          # (q tiles x heads) from which a launch plan is built for a single call
PLAN_MIN_ITEMS_SHARED = 1024   # ... when a LaunchPlan object shares it between calls


class LaunchPlan:
    """Keeps the launch plan of one packed batch so that calls with the same lengths share it.

    Pass one object as ``launch_plan=`` to every ``flash_attention_with_fusing_bias_varlen`` call over
    the same batch (the layers of a stack): the first call builds the plan on the device, the others
    find the workspace ready.  The object compares the identity and version of the length tensors
    (int32 device tensors, which it keeps alive) and the launch shape, and rebuilds when they differ;
    lengths changed behind torch's back (a raw kernel writing into the same tensor) go unnoticed.
    Use one object per stream.
    """

    def __init__(self):
        self.key = None
        self.tensors = None     # the length tensors of the key, kept alive: their addresses cannot be reused
        self.workspace = None

    def lookup(self, key, tensors, nbytes, device):
        """-> (workspace, ready).  A plan that is not ready counts as built only after ``commit``."""
        if self.key == key and self.workspace is not None:
            return self.workspace, True
        if self.workspace is None or self.workspace.numel() < nbytes or self.workspace.device != device:
            self.workspace = torch.empty(nbytes, device=device, dtype=torch.uint8)
        self.key, self.tensors = None, None
        return self.workspace, False

    def commit(self, key, tensors):
        """The library has queued the build for ``key`` (its call returned without error)."""
        self.key, self.tensors = key, tensors


def _varlen_forward(q, k, v, bias, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale, NUM_BUCKETS,
                    MAX_DISTANCE, return_lse, seq_lens_q, seq_lens_k, launch_plan, exact_scores):
    _check_inputs(q, k, v)
    total_q, H, D = q.shape
    total_k = k.shape[0]
    if k.shape[1] != H or v.shape != k.shape:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    B = cu_seqlens_q.numel() - 1
    if cu_seqlens_k.numel() != B + 1:
        raise ValueError("cu_seqlens_q and cu_seqlens_k must have the same length")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    cq = cu_seqlens_q.to(device=q.device, dtype=torch.int32).contiguous()
    ck = cq if cu_seqlens_k is cu_seqlens_q else cu_seqlens_k.to(device=q.device, dtype=torch.int32).contiguous()
    q_, k_, v_ = (_kernel_ready(t) for t in (q, k, v))
    lens = []
    for t in (seq_lens_q, seq_lens_k):
        if t is not None:
            if t.numel() != B:
                raise ValueError(f"seq_lens must hold {B} lengths, got {t.numel()}")
            t = t.to(device=q.device, dtype=torch.int32).contiguous()
        lens.append(t)
    # padding rows are not written by the kernel: they read as zeros, like the reference's pad_input
    o = torch.empty_like(q_) if lens[0] is None else torch.zeros_like(q_)
    lse = None
    if return_lse:
        lse = (torch.empty if lens[0] is None else torch.zeros)((total_q, H), device=q.device, dtype=torch.float32)
    a = L.T5AVarlenArgs()
    a.q, a.k, a.v, a.o = q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr()
    a.lse = lse.data_ptr() if lse is not None else None
    for name, t in (("q_strides", q_), ("k_strides", k_), ("v_strides", v_), ("o_strides", o)):
        setattr(a, name, (C.c_int64 * 2)(t.stride(0), t.stride(1)))
    a.cu_seqlens_q, a.cu_seqlens_k = cq.data_ptr(), ck.data_ptr()
    a.seq_lens_q = lens[0].data_ptr() if lens[0] is not None else None
    a.seq_lens_k = lens[1].data_ptr() if lens[1] is not None else None
    a.dtype, a.B, a.H, a.D = _dtype_code(q), B, H, D
    a.total_q, a.total_k = total_q, total_k
    a.max_seqlen_q, a.max_seqlen_k = int(max_seqlen_q), int(max_seqlen_k)
    a.causal, a.sm_scale = int(bool(causal)), float(sm_scale)
    a.exact_scores = _exact(exact_scores)
    a.bias, keep = _bias_struct(bias, H, NUM_BUCKETS, MAX_DISTANCE, q, causal)
    lib = L.load()
    # building a plan costs about 15 us: worth it from a few thousand items on, earlier when shared
    items = (total_q // 128 + B) * H
    shared = isinstance(launch_plan, LaunchPlan)
    wanted = launch_plan == "always" or (shared and items >= PLAN_MIN_ITEMS_SHARED) or \
        (launch_plan is True and items >= PLAN_MIN_ITEMS)
    ws_bytes = lib.t5a_varlen_workspace_bytes(B, H, total_q) if wanted else 0
    plan_key = None
    if ws_bytes > 0:
        # under graph capture nothing runs yet: a plan recorded there must not count as built for later eager calls
        if shared and not torch.cuda.is_current_stream_capturing():
            key = tuple((t.data_ptr(), t._version) if t is not None else None for t in (cq, ck, lens[0], lens[1]))
            key += (B, H, D, total_q, a.dtype, a.causal, a.max_seqlen_q, a.max_seqlen_k, str(q.device))
            ws, ready = launch_plan.lookup(key, (cq, ck, lens[0], lens[1]), ws_bytes, q.device)
            a.workspace_ready = int(ready)
            if not ready:
                plan_key = key
        else:
            ws = torch.empty(ws_bytes, device=q.device, dtype=torch.uint8)   # stream-ordered reuse by torch's allocator
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws_bytes
    with _on_device(q):
        L.check(lib.t5a_fwd_varlen(C.byref(a), _stream(q)))
    launched = B > 0 and total_q > 0
    _commit_lut(keep, launched)
    if plan_key is not None and launched:
        launch_plan.commit(plan_key, (cq, ck, lens[0], lens[1]))
    return (o, lse) if return_lse else o


def _varlen_backward(q, k, v, bias, o, lse, dout, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale,
                     NUM_BUCKETS, MAX_DISTANCE, seq_lens_q, seq_lens_k, exact_scores):
    """-> dq, dk, dv, dbias (fp32 (NUM_BUCKETS, H) or None); t5a_bwd_varlen"""
    total_q, H, D = q.shape
    if D == 128 and (q.dtype == torch.float32 or BACKWARD_FP32_MATH):
        raise NotImplementedError("backward at head_dim 128: bf16 / fp16 tensors only (the fp32 kernels cover head_dim 16, 32 and 64)")
    B = cu_seqlens_q.numel() - 1
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    cq = cu_seqlens_q.to(device=q.device, dtype=torch.int32).contiguous()
    ck = cq if cu_seqlens_k is cu_seqlens_q else cu_seqlens_k.to(device=q.device, dtype=torch.int32).contiguous()
    lens = [t.to(device=q.device, dtype=torch.int32).contiguous() if t is not None else None for t in (seq_lens_q, seq_lens_k)]
    q_, k_, v_, o_, g_ = (_kernel_ready(t) for t in (q, k, v, o, dout))
    # rows of padding (between a sequence's length and the next sequence's first row) get no gradient
    dq = (torch.empty_like if lens[0] is None else torch.zeros_like)(q_)
    dk = (torch.empty_like if lens[1] is None else torch.zeros_like)(k_)
    dv = (torch.empty_like if lens[1] is None else torch.zeros_like)(v_)
    dtable = torch.empty((NUM_BUCKETS, H), device=q.device, dtype=torch.float32) if bias is not None else None
    lib = L.load()
    ws = torch.empty(max(int(lib.t5a_bwd_varlen_workspace_bytes(total_q, H)), 16), device=q.device, dtype=torch.uint8)
    a = L.T5AVarlenBwdArgs()
    a.q, a.k, a.v, a.o, a.dout, a.lse = (t.data_ptr() for t in (q_, k_, v_, o_, g_, lse))
    a.dq, a.dk, a.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    a.dtable = dtable.data_ptr() if dtable is not None else None
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    for name, t in (("q_strides", q_), ("k_strides", k_), ("v_strides", v_), ("o_strides", o_), ("dout_strides", g_),
                    ("dq_strides", dq), ("dk_strides", dk), ("dv_strides", dv)):
        setattr(a, name, (C.c_int64 * 2)(t.stride(0), t.stride(1)))
    a.cu_seqlens_q, a.cu_seqlens_k = cq.data_ptr(), ck.data_ptr()
    a.seq_lens_q = lens[0].data_ptr() if lens[0] is not None else None
    a.seq_lens_k = lens[1].data_ptr() if lens[1] is not None else None
    a.dtype, a.B, a.H, a.D = _dtype_code(q), B, H, D
    a.total_q, a.total_k = total_q, k.shape[0]
    a.max_seqlen_q, a.max_seqlen_k = int(max_seqlen_q), int(max_seqlen_k)
    a.causal, a.sm_scale = int(bool(causal)), float(sm_scale)
    a.exact_scores = _exact(exact_scores)
    a.fp32_math = int(bool(BACKWARD_FP32_MATH))
    b = L.T5ABias()
    table = None
    if bias is not None:
        table = bias.detach()
        if table.dtype not in _DTYPES:
            table = table.float()
        b.table, b.table_dtype = table.data_ptr(), _DTYPES[table.dtype]
        b.num_buckets, b.max_distance = NUM_BUCKETS, MAX_DISTANCE
        b.stride_bucket, b.stride_head = table.stride(0), table.stride(1)
    a.bias = b
    with _on_device(q):
        L.check(lib.t5a_bwd_varlen(C.byref(a), _stream(q)))
    del table
    return dq, dk, dv, dtable


class FlashAttentionBiasVarlen(torch.autograd.Function):
    """The packed forward with its backward (reference varlen_fused_bias_attn.py:800-868)."""

    @staticmethod
    def forward(ctx, q, k, v, bias, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale, NUM_BUCKETS,
                MAX_DISTANCE, seq_lens_q, seq_lens_k, launch_plan, exact_scores):
        o, lse = _varlen_forward(q, k, v, bias, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale,
                                 NUM_BUCKETS, MAX_DISTANCE, True, seq_lens_q, seq_lens_k, launch_plan, exact_scores)
        ctx.save_for_backward(q, k, v, o, lse, *(() if bias is None else (bias,)))
        ctx.has_bias = bias is not None
        ctx.args = (cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, bool(causal), sm_scale, NUM_BUCKETS, MAX_DISTANCE,
                    seq_lens_q, seq_lens_k, exact_scores)
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, dout, _dlse):
        q, k, v, o, lse = ctx.saved_tensors[:5]
        bias = ctx.saved_tensors[5] if ctx.has_bias else None
        cq, ck, mq, mk, causal, sm_scale, nb, md, lq, lk, exact = ctx.args
        dq, dk, dv, dtable = _varlen_backward(q, k, v, bias, o, lse, dout, cq, ck, mq, mk, causal, sm_scale, nb, md, lq, lk, exact)
        dbias = dtable.to(bias.dtype) if bias is not None and ctx.needs_input_grad[3] else None
        return (dq, dk, dv, dbias) + (None,) * 12


def flash_attention_with_fusing_bias_varlen(q, k, v, bias, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                            causal=False, sm_scale=None, NUM_BUCKETS=32, MAX_DISTANCE=128,
                                            return_lse: bool = False, seq_lens_q=None, seq_lens_k=None,
                                            launch_plan: bool = True, exact_scores: Optional[bool] = None):
    """Packed variable-length forward: q (total_q,H,D), k/v (total_k,H,D), cu_seqlens int32 on the device.

    Positions restart at 0 in every sequence.  No host synchronisation: the
    work list is derived on the device from ``cu_seqlens``.

    ``seq_lens_q`` / ``seq_lens_k`` (optional int32 device tensors of B lengths): sequence b is rows
    [cu[b], cu[b] + lens[b]); the rows up to cu[b+1] are padding, never read and left ZERO in the
    output.  A right-padded (B, L, H, D) batch runs in place this way, viewed as (B*L, H, D) with
    cu = arange(B+1) * L and lens = mask.sum(-1): no gathers, no scatter.

    ``launch_plan``: True (default) lets larger launches first build, on the device, per-XCD item
    lists of equal work from ``cu_seqlens`` (a small workspace is taken from torch's allocator);
    False never does, ``"always"`` does whatever the size.  A ``LaunchPlan`` object keeps the plan
    for later calls over the same batch.  The results do not depend on any of this.
    """
    needs_grad = torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (q, k, v, bias))
    if needs_grad:
        o, lse = FlashAttentionBiasVarlen.apply(q, k, v, bias, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal,
                                                sm_scale, NUM_BUCKETS, MAX_DISTANCE, seq_lens_q, seq_lens_k, launch_plan,
                                                exact_scores)
        return (o, lse) if return_lse else o
    return _varlen_forward(q, k, v, bias, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale,
                           NUM_BUCKETS, MAX_DISTANCE, return_lse, seq_lens_q, seq_lens_k, launch_plan, exact_scores)


KEY_BITS_FRONT = 8   # zero words in front of a sequence's validity bits (kKeyBitsFront of the library)


def pack_key_bits(attention_mask: torch.Tensor, block_len: int, aux: int = 0) -> torch.Tensor:
    """(B, L) mask (non-zero = token) -> (B, words) int32 bit sets as ``t5a_sparse_args.key_bits`` wants them: token j
    is bit (j & 31) of word 8 + (j >> 5), zero words in front and behind.  Runs on the mask's device, no host sync."""
    if attention_mask.dim() != 2:
        raise ValueError("attention_mask must be (B, L)")
    B, Lm = attention_mask.shape
    words = int(L.load().t5a_sparse_key_bits_words(Lm, int(block_len), int(aux)))
    body = (Lm + 31) // 32
    valid = (attention_mask != 0)
    if body * 32 != Lm:
        valid = torch.nn.functional.pad(valid, (0, body * 32 - Lm))
    weights = (torch.ones(32, dtype=torch.int64, device=valid.device) << torch.arange(32, device=valid.device))
    packed = (valid.view(B, body, 32).to(torch.int64) * weights).sum(-1)            # 0 .. 2^32 - 1
    packed = torch.where(packed >= 2 ** 31, packed - 2 ** 32, packed).to(torch.int32)
    out = torch.zeros(B, words, dtype=torch.int32, device=valid.device)
    out[:, KEY_BITS_FRONT:KEY_BITS_FRONT + body] = packed
    return out


def side_token_counts(attention_mask: torch.Tensor, global_block_size: int) -> torch.Tensor:
    """(B, L) mask -> (B,) int32: the side tokens of each sequence, one per valid token at the END of a block of
    ``global_block_size`` positions (src/turbot5/model/utils.py:206-216).  On the mask's device, no host sync."""
    g = int(global_block_size)
    return (attention_mask[:, g - 1::g] != 0).sum(-1).to(torch.int32).contiguous()


def _sparse(pattern, q, k, v, bias, block_len, aux, side_k=None, side_v=None, sm_scale=1.0,
            NUM_BUCKETS=32, MAX_DISTANCE=128, key_splits=True, seq_lens=None, exact_scores=None, seq_starts=None,
            key_bits=None, side_counts=None):
    _check_inputs(q, k, v)
    _forward_only("sparse attention (local, block, transient-global)", q, k, v, bias, side_k, side_v)
    B, H, Lq, D = q.shape
    if side_counts is not None and (pattern != L.PATTERN_TGLOBAL or key_bits is None):
        raise ValueError("side_counts goes with key_bits in the transient-global pattern")
    if key_bits is not None:
        if seq_lens is not None:
            raise ValueError("key_bits is instead of seq_lens")
        if pattern == L.PATTERN_TGLOBAL and (side_counts is None or side_counts.dtype != torch.int32 or side_counts.shape != (B,)
                                             or side_counts.device != q.device or not side_counts.is_contiguous()):
            raise ValueError("transient-global attention with key_bits needs side_counts: side_token_counts(mask, global_block_size)")
        need = int(L.load().t5a_sparse_key_bits_words(Lq, int(block_len), int(aux)))
        if (key_bits.dtype != torch.int32 or key_bits.dim() != 2 or key_bits.shape[0] != B or key_bits.shape[1] < need
                or key_bits.device != q.device or not key_bits.is_contiguous()):
            raise ValueError(f"key_bits must be a contiguous int32 tensor (B, >= {need}) on the device of q: pack_key_bits()")
    for name, t in (("seq_lens", seq_lens), ("seq_starts", seq_starts)):
        if t is not None and (t.dtype != torch.int32 or t.shape != (B,) or t.device != q.device or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous int32 tensor of shape (B,) on the device of q")
    if seq_starts is not None and (seq_lens is None or pattern == L.PATTERN_BLOCK):
        raise ValueError("seq_starts needs seq_lens and the local or transient-global pattern")
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("sparse self-attention needs q, k, v of one shape")
    q_, k_, v_ = (_kernel_ready(t) for t in (q, k, v))
    o = torch.empty_like(q_)
    a = L.T5ASparseArgs()
    a.q, a.k, a.v, a.o = q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr()
    a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides3(q_), _strides3(k_), _strides3(v_), _strides3(o)
    keep_side = None
    if pattern == L.PATTERN_TGLOBAL:
        if side_k is None or side_v is None or side_k.shape != side_v.shape:
            raise ValueError("transient-global attention needs side_k and side_v of one shape")
        if side_k.shape[0] != B or side_k.shape[1] != H or side_k.shape[3] != D or side_k.dtype != q.dtype:
            raise ValueError(f"side_k must be (B,H,n_side,D) in {q.dtype}, got {tuple(side_k.shape)} {side_k.dtype}")
        sk, sv = _kernel_ready(side_k.detach()), _kernel_ready(side_v.detach())
        keep_side = (sk, sv)
        a.side_k, a.side_v = sk.data_ptr(), sv.data_ptr()
        a.side_k_strides, a.side_v_strides = _strides3(sk), _strides3(sv)
        a.n_side = sk.shape[2]
    a.dtype, a.B, a.H, a.L, a.D = _dtype_code(q), B, H, Lq, D
    a.pattern, a.block_len, a.aux = pattern, int(block_len), int(aux)
    a.sm_scale = float(sm_scale)
    a.exact_scores = _exact(exact_scores)
    a.run_len = int(RUN_LEN)
    if seq_lens is not None:
        a.seq_lens = seq_lens.data_ptr()
    if seq_starts is not None:
        a.seq_starts = seq_starts.data_ptr()
    if key_bits is not None:
        a.key_bits, a.key_bits_stride = key_bits.data_ptr(), key_bits.shape[1]
        if side_counts is not None:
            a.side_counts = side_counts.data_ptr()
    # the local pattern's work items fetch LUT images that have the window folded in (windows up to 256)
    window = int(block_len) if pattern == L.PATTERN_LOCAL and int(block_len) <= 256 and key_bits is None else 0
    a.bias, keep = _bias_struct(bias, H, NUM_BUCKETS, MAX_DISTANCE, q, window=window)
    lib = L.load()
    ws_bytes = lib.t5a_sparse_workspace_bytes(pattern, B, H, Lq, D, int(block_len), int(aux))
    workspace = None
    if ws_bytes > 0 and key_splits:   # block pattern: key splits of the global rows
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), ws_bytes
    with _on_device(q):
        L.check(lib.t5a_fwd_sparse(C.byref(a), _stream(q)))
    _commit_lut(keep, B > 0 and Lq > 0)
    return o


def local_attention_with_fusing_bias(q, k, v, bias, block_len, sm_scale=1.0, NUM_BUCKETS=32, MAX_DISTANCE=128,
                                     seq_lens=None, exact_scores=None, seq_starts=None, key_bits=None):
    """Sliding-window self-attention: key j visible to query i iff |j-i| < block_len, bias bucket(j-i).

    The op of T5LocalAttention (src/turbot5/model/attentions.py:583-638) without
    blocking, K/V triplication or a bias tensor.  q,k,v (B,H,L,D).
    ``seq_lens`` / ``seq_starts`` (B,) int32: the tokens of sequence b are the rows [start, start + len) (start
    defaults to 0: right padding); keys outside them are not attended (the mask of
    src/turbot5/model/utils.py:174-188 for the sequence's own rows), positions stay the row indices.
    ``key_bits`` (``pack_key_bits(mask, block_len)``, instead of seq_lens): the same for a mask of any shape."""
    return _sparse(L.PATTERN_LOCAL, q, k, v, bias, block_len, 0, None, None, sm_scale, NUM_BUCKETS, MAX_DISTANCE,
                   seq_lens=seq_lens, exact_scores=exact_scores, seq_starts=seq_starts, key_bits=key_bits)


def block_attention_with_fusing_bias(q, k, v, bias, block_len, n_global, sm_scale=1.0, NUM_BUCKETS=32,
                                     MAX_DISTANCE=128, key_splits=True, exact_scores=None, seq_lens=None, key_bits=None):
    """Block attention with ``n_global`` leading global tokens, the op of T5BlockAttention
    (src/turbot5/model/attentions.py:788-853) with the reference's key/mask layout.

    ``key_splits``: hand the library a workspace so that the global rows (which attend every key) are
    spread over the device as key splits and merged; False keeps them in one workgroup per (batch, head).
    ``seq_lens`` (B,) int32: valid tokens of each right-padded sequence, masked the way the reference lays its
    padding mask over the key list (attentions.py:722-732); the global rows see every key regardless (:788-800).
    ``key_bits`` (``pack_key_bits(mask, block_len, n_global)``): the same for a mask of any shape."""
    return _sparse(L.PATTERN_BLOCK, q, k, v, bias, block_len, n_global, None, None, sm_scale, NUM_BUCKETS,
                   MAX_DISTANCE, key_splits=key_splits, exact_scores=exact_scores, seq_lens=seq_lens, key_bits=key_bits)


def transient_global_attention_with_fusing_bias(q, k, v, side_k, side_v, bias, block_len, global_block_size,
                                                sm_scale=1.0, NUM_BUCKETS=32, MAX_DISTANCE=128, seq_lens=None,
                                                exact_scores=None, seq_starts=None, key_bits=None, side_counts=None):
    """Sliding window plus side tokens, the op of T5TransientGlobalAttention
    (src/turbot5/model/attentions.py:977-1052).  side_k/side_v (B,H,L//global_block_size,D).
    ``seq_lens`` / ``seq_starts`` (B,) int32: the tokens of sequence b are the rows [start, start + len); it has
    (start + len) // global_block_size - start // global_block_size side tokens
    (src/turbot5/model/utils.py:191-237 for one run of tokens) and only its own rows as keys.
    ``key_bits`` (``pack_key_bits(mask, block_len, global_block_size)``) with ``side_counts``
    (``side_token_counts(mask, global_block_size)``), instead of seq_lens: the same for a mask of any shape."""
    return _sparse(L.PATTERN_TGLOBAL, q, k, v, bias, block_len, global_block_size, side_k, side_v, sm_scale,
                   NUM_BUCKETS, MAX_DISTANCE, seq_lens=seq_lens, exact_scores=exact_scores, seq_starts=seq_starts,
                   key_bits=key_bits, side_counts=side_counts)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, group: int = 1,
             residual: Optional[torch.Tensor] = None, seq_lens: Optional[torch.Tensor] = None,
             seq_starts: Optional[torch.Tensor] = None, key_bits: Optional[torch.Tensor] = None,
             group_counts: Optional[torch.Tensor] = None):
    """T5 RMS norm over the last dimension (src/turbot5/model/modules.py:51-59).

    With ``residual`` (same shape and dtype as x, group 1) the kernel normalises ``x + residual`` and
    returns ``(x + residual, norm)``: the residual add that ends one T5 sub-layer and the norm that
    opens the next (src/turbot5/model/modeling.py:159-161, :113-114) in one pass.

    ``group`` > 1: x is (B, L, d) and row r of the (B, L // group, d) result is the norm of the sum of
    rows [r*group, (r+1)*group) of its sequence, trailing rows joining the last group: the side-token
    producer of transient-global attention (src/turbot5/model/utils.py:249-258, :206-212).
    ``seq_lens`` / ``seq_starts`` (B,) int32 for x of shape (B, L, d), not together with ``residual``: the rows
    [start, start + len) of each sequence are its tokens (start defaults to 0); it has one group per group end among
    them, the last group taking every token from its first row on; output rows past the groups are zero.
    ``key_bits`` with ``group_counts`` (``pack_key_bits``, ``side_token_counts``), instead of seq_lens: the same for a
    mask of any shape -- a group sums its valid rows.
    The result has the weight's dtype when that is 16 bit, else fp32, as torch promotes the reference code."""
    if not (x.is_cuda and weight.is_cuda):
        raise RuntimeError("x and weight must be on a ROCm device: this path has no CPU implementation")
    d = x.shape[-1]
    if weight.shape != (d,):
        raise ValueError(f"weight must have shape ({d},), got {tuple(weight.shape)}")
    out_dtype = weight.dtype if weight.dtype in (torch.float16, torch.bfloat16) else torch.float32
    w = weight.detach().contiguous()
    x_ = x.detach()
    r2 = None
    if residual is not None:
        if group != 1 or residual.shape != x.shape or residual.dtype != x.dtype or residual.device != x.device:
            raise ValueError("residual needs group == 1 and the shape, dtype and device of x")
        r2 = residual.detach().reshape(-1, d)
        if r2.stride(-1) != 1 or r2.stride(0) % 8 != 0 or r2.data_ptr() % 16 != 0:
            r2 = r2.contiguous()
    if group == 1 and seq_lens is None:
        x2 = x_.reshape(-1, d)
        if x2.stride(-1) != 1 or x2.stride(0) % 8 != 0 or x2.data_ptr() % 16 != 0:
            x2 = x2.contiguous()
        batches, rows, strides = 1, x2.shape[0], (0, x2.stride(0))
        out_shape = x.shape
    else:
        if x_.dim() != 3:
            raise ValueError("grouped rms_norm needs x of shape (B, L, d)")
        x2 = x_
        if x2.stride(-1) != 1 or x2.stride(0) % 8 != 0 or x2.stride(1) % 8 != 0 or x2.data_ptr() % 16 != 0:
            x2 = x2.contiguous()
        batches, rows, strides = x2.shape[0], x2.shape[1], (x2.stride(0), x2.stride(1))
        out_shape = (x2.shape[0], rows // group, d)
    y = torch.empty(out_shape, dtype=out_dtype, device=x.device)
    a = L.T5ARmsNormArgs()
    a.x, a.weight, a.y = x2.data_ptr(), w.data_ptr(), y.data_ptr()
    a.x_strides = (C.c_int64 * 2)(*strides)
    a.batches, a.rows_per_batch, a.dim, a.group = batches, rows, d, int(group)
    a.x_dtype, a.weight_dtype, a.eps = _dtype_code(x2), _dtype_code(w), float(eps)
    if seq_lens is not None:
        if residual is not None or seq_lens.dtype != torch.int32 or seq_lens.shape != (batches,) \
                or seq_lens.device != x.device or not seq_lens.is_contiguous():
            raise ValueError("seq_lens must be a contiguous int32 tensor of shape (B,) on the device of x, without residual")
        a.seq_lens = seq_lens.data_ptr()
        if seq_starts is not None:
            if seq_starts.dtype != torch.int32 or seq_starts.shape != (batches,) or seq_starts.device != x.device \
                    or not seq_starts.is_contiguous():
                raise ValueError("seq_starts must be a contiguous int32 tensor of shape (B,) on the device of x")
            a.seq_starts = seq_starts.data_ptr()
    elif seq_starts is not None:
        raise ValueError("seq_starts needs seq_lens")
    if key_bits is not None or group_counts is not None:
        need = KEY_BITS_FRONT + (rows + 31) // 32
        if (key_bits is None or group_counts is None or group <= 1 or seq_lens is not None or residual is not None
                or key_bits.dtype != torch.int32 or key_bits.dim() != 2 or key_bits.shape[0] != batches or key_bits.shape[1] < need
                or key_bits.device != x.device or not key_bits.is_contiguous()
                or group_counts.dtype != torch.int32 or group_counts.shape != (batches,) or group_counts.device != x.device
                or not group_counts.is_contiguous()):
            raise ValueError(f"key_bits (B, >= {need}) int32 and group_counts (B,) int32 go together, contiguous on the device "
                             "of x, with group > 1 and without seq_lens or residual")
        a.key_bits, a.key_bits_stride, a.group_counts = key_bits.data_ptr(), key_bits.shape[1], group_counts.data_ptr()
    total = None
    if r2 is not None:
        total = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        a.residual, a.sum_out, a.residual_row_stride = r2.data_ptr(), total.data_ptr(), r2.stride(0)
    with _on_device(x):
        L.check(L.load().t5a_rmsnorm(C.byref(a), _stream(x)))
    return y if total is None else (total, y)


_CU_COUNT = {}


def _cu_count(device) -> int:
    if device is None or not torch.cuda.is_available():
        return 256
    idx = torch.device(device).index
    if idx not in _CU_COUNT:
        _CU_COUNT[idx] = torch.cuda.get_device_properties(device).multi_processor_count
    return _CU_COUNT[idx]


def default_num_splits(B: int, H: int, N: int, device=None) -> int:
    """Some 48 workgroups per compute unit, at least 512 keys per split: many short workgroups keep every
    HBM channel busy to the end (B64 H12 over 8192 keys: 16 splits 6.0 TB/s, 2 splits 5.75, measured)."""
    cus = _cu_count(device)
    want = max(1, (48 * cus + B * H - 1) // max(1, B * H))
    return int(max(1, min(want, max(1, N // 512), 64)))


def flash_attn_v2_fwd(q, k, v, bias, causal, sm_scale, NUM_SPLITS=None, BLOCK_M=None, BLOCK_N=None, num_warps=None,
                      num_stages=None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Flash-decoding split-K forward (src/turbot5/ops/flash_decoding.py:6-55).

    q (B,H,M,D) with small M; k, v (B,H,N,D); ``bias`` an additive tensor
    broadcastable to (B,H,M,N) or None; ``causal`` is accepted and unused, as in
    the reference; the tile arguments are accepted and ignored (fixed in the
    kernel).  Returns (res, L, ml): res (B,H,M,D) fp32 merged output, L and ml
    the per-split sums of exp and maxima, (B,H,S) when M == 1 else (B,H,S,M).
    """
    out, part_l, part_m = _splitk(q, k, v, bias, sm_scale, NUM_SPLITS, out_dtype=torch.float32)
    if q.shape[2] == 1:
        part_l, part_m = part_l.squeeze(-1), part_m.squeeze(-1)
    return out, part_l, part_m


def flash_decoding_attention(q, k, v, bias=None, sm_scale=1.0, num_splits=None, key_lens=None,
                             key_starts=None) -> torch.Tensor:
    """Split-K attention returning only the merged output in q's dtype.

    ``key_lens`` / ``key_starts`` (optional (B,) int32 device tensors): batch element b only has the keys
    [start, start + len) of its N rows -- a padded encoder memory, which the reference masks with an additive
    bias (src/turbot5/model/attentions.py:235-236).  Rows of a batch element without keys come out zero."""
    return _splitk(q, k, v, bias, sm_scale, num_splits, out_dtype=q.dtype, key_lens=key_lens, key_starts=key_starts)[0]


def flash_decoding_attention_static(q, k, v, out, sm_scale=1.0, num_splits=None, key_lens=None, key_starts=None):
    """Split-K attention that allocates nothing: the caller passes the (B,H,M,D) output tensor and the partial
    results go to the library's static scratch array (``t5a_fwd_splitk_static``).  For callers that cannot
    allocate, such as code under graph capture.  q, k, v must already be kernel-ready (head_dim contiguous,
    16-byte aligned rows); B*H*num_splits*M*(D+2)*4 bytes must fit ``_lib.STATIC_SCRATCH_BYTES``.  Calls that
    overlap in time on one GPU race on the shared array; calls ordered on one stream do not."""
    _check_inputs(q, k, v)
    B, H, M, D = q.shape
    N = k.shape[2]
    if out.shape != q.shape or out.dtype != q.dtype or out.device != q.device:
        raise ValueError("out must have the shape, dtype and device of q")
    for t in (q, k, v):
        if _kernel_ready(t) is not t:
            raise ValueError("q, k, v must have head_dim contiguous and 16-byte aligned rows (no copies are made here)")
    S = int(num_splits) if num_splits else default_num_splits(B, H, N, q.device)
    a = L.T5ASplitKArgs()
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides3(q), _strides3(k), _strides3(v), _strides3(out)
    a.dtype, a.B, a.H, a.M, a.N, a.D = _dtype_code(q), B, H, M, N, D
    a.num_splits, a.sm_scale = S, float(sm_scale)
    if key_lens is not None:
        a.key_lens = key_lens.data_ptr()
        a.key_starts = key_starts.data_ptr() if key_starts is not None else None
    with _on_device(q):
        L.check(L.load().t5a_fwd_splitk_static(C.byref(a), _stream(q)))
    return out


def _splitk(q, k, v, bias, sm_scale, num_splits, out_dtype, key_lens=None, key_starts=None):
    _check_inputs(q, k, v)
    B, H, M, D = q.shape
    for name, t in (("key_lens", key_lens), ("key_starts", key_starts)):
        if t is not None and (t.dtype != torch.int32 or t.shape != (B,) or t.device != q.device or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous int32 tensor of shape (B,) on the device of q")
    if key_starts is not None and key_lens is None:
        raise ValueError("key_starts needs key_lens")
    N = k.shape[2]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    S = int(num_splits) if num_splits else default_num_splits(B, H, N, q.device)
    q_, k_, v_ = (_kernel_ready(t) for t in (q, k, v))
    lib = L.load()
    nbytes = lib.t5a_splitk_workspace_bytes(B, H, M, D, S)
    ws = torch.empty(max(nbytes, 16) // 4, device=q.device, dtype=torch.float32)
    o = torch.empty((B, H, M, D), device=q.device, dtype=q.dtype)
    a = L.T5ASplitKArgs()
    a.q, a.k, a.v, a.o = q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr()
    a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides3(q_), _strides3(k_), _strides3(v_), _strides3(o)
    keep = None
    if bias is not None:
        keep = bias.detach().float().expand(B, H, M, N)
        a.attn_bias = keep.data_ptr()
        a.bias_strides = (C.c_int64 * 4)(*keep.stride())
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel() * 4
    a.dtype, a.B, a.H, a.M, a.N, a.D = _dtype_code(q), B, H, M, N, D
    a.num_splits, a.sm_scale = S, float(sm_scale)
    if key_lens is not None:
        a.key_lens = key_lens.data_ptr()
        a.key_starts = key_starts.data_ptr() if key_starts is not None else None
    with _on_device(q):
        L.check(lib.t5a_fwd_splitk(C.byref(a), _stream(q)))
    rows = B * H * S * M
    part_l = ws[rows * D: rows * D + rows].view(B, H, S, M)
    part_m = ws[rows * D + rows: rows * D + 2 * rows].view(B, H, S, M)
    return (o if out_dtype == q.dtype else o.to(out_dtype)), part_l, part_m
