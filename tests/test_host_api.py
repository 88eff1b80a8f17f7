"""CPU-only checks of the boundary: the C-ABI library loads and exports what include/t5attn.h
declares, argument validation works without a GPU, the host bucket table equals the oracle's, and
the module surface mirrors the reference's."""
import ctypes as C
import inspect
import os
import re

import pytest
import torch

from oracle import t5_basic as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from turbot5_amd import _lib
    return _lib


def test_header_symbols_are_exported(lib):
    header = open(os.path.join(ROOT, "include", "t5attn.h")).read()
    declared = set(re.findall(r"\b(t5a_[a-z_0-9]+)\s*\(", header))
    assert declared == set(lib.EXPORTS)
    handle = lib.load()
    for name in declared:
        assert getattr(handle, name) is not None
    assert handle.t5a_version() == lib.ABI_VERSION == int(re.search(r"#define T5A_ABI_VERSION (\d+)", header).group(1))


def test_struct_sizes_follow_the_header(lib):
    # natural alignment, no packing: catches a field added on one side only
    assert C.sizeof(lib.T5ABias) == 8 + 4 * 4 + 2 * 8 + 2 * 8 + 2 * 4
    assert C.sizeof(lib.T5ADenseArgs) == 5 * 8 + 12 * 8 + 10 * 4 + C.sizeof(lib.T5ABias)
    assert C.sizeof(lib.T5AVarlenArgs) == 5 * 8 + 8 * 8 + 4 * 8 + 2 * 8 + 12 * 4 + C.sizeof(lib.T5ABias)
    assert C.sizeof(lib.T5ASparseArgs) == 8 * 8 + 18 * 8 + 11 * 4 + 4 + C.sizeof(lib.T5ABias) + 5 * 8 + 2 * 4
    assert C.sizeof(lib.T5ASplitKArgs) == 7 * 8 + 16 * 8 + 8 * 4 + 2 * 8
    assert C.sizeof(lib.T5ARmsNormArgs) == 3 * 8 + 2 * 8 + 8 + 8 * 4 + 5 * 8 + 3 * 8


def test_key_bits_layout_and_size(lib):
    """Token j is bit (j & 31) of word 8 + (j >> 5); zero words in front and behind, as many as the kernels' tiles
    may look at; the side-token count is the number of valid block ENDs."""
    from turbot5_amd import ops
    handle = lib.load()
    assert handle.t5a_sparse_key_bits_words(1000, 128, 16) == 8 + (1000 + 256 + 16 + 256 + 31) // 32 + 4
    assert handle.t5a_sparse_key_bits_words(-1, 128, 0) == -1 and handle.t5a_sparse_key_bits_words(10, 0, 0) == -1
    g = torch.Generator().manual_seed(5)
    for Lm in (1, 31, 32, 33, 100, 257):
        mask = (torch.rand(3, Lm, generator=g) > 0.4).float()
        mask[2] = 1
        bits = ops.pack_key_bits(mask, 64, 8)
        assert bits.dtype == torch.int32 and bits.shape == (3, handle.t5a_sparse_key_bits_words(Lm, 64, 8))
        words = bits.to(torch.int64) & 0xFFFFFFFF
        for b in range(3):
            for j in range(Lm):
                assert (int(words[b, ops.KEY_BITS_FRONT + (j >> 5)]) >> (j & 31)) & 1 == int(mask[b, j]), (Lm, b, j)
        assert (words[:, :ops.KEY_BITS_FRONT] == 0).all()
        tail = words[:, ops.KEY_BITS_FRONT + (Lm + 31) // 32:]
        assert (tail == 0).all()
        if Lm % 32:   # bits past the last token stay zero
            assert (int(words[2, ops.KEY_BITS_FRONT + Lm // 32]) >> (Lm % 32)) == 0
    mask = torch.ones(2, 50)
    mask[0, 15] = 0
    mask[1, 40:] = 0
    assert ops.side_token_counts(mask, 16).tolist() == [2, 2]
    assert ops.side_token_counts(mask, 8).tolist() == [5, 5]


@pytest.mark.parametrize("bidirectional", [True, False])
@pytest.mark.parametrize("nb,md", [(32, 128), (64, 256), (16, 64), (32, 20), (128, 512), (8, 1000), (256, 300)])
def test_bucket_lut_equals_oracle(lib, bidirectional, nb, md):
    got = lib.bucket_lut(bidirectional, nb, md)
    rel = torch.arange(-md, md + 1)
    want = O.relative_position_bucket(rel, bidirectional, nb, md).tolist()
    assert got == want


def test_bucket_lut_rejects_bad_parameters(lib):
    for args in ((True, 2, 128), (False, 1, 128), (True, 32, 8), (True, 2048, 100000)):
        with pytest.raises(lib.T5AError) as e:
            lib.bucket_lut(*args)
        assert e.value.code == -6


def test_validation_without_gpu(lib):
    handle = lib.load()
    a = lib.T5ADenseArgs()
    a.dtype, a.B, a.H, a.M, a.N, a.D = 0, 1, 1, 8, 8, 48
    assert handle.t5a_fwd_dense(C.byref(a), None) == -3          # head dim
    assert b"head_dim" in handle.t5a_last_error()
    a.D = 64
    a.dtype = 7
    assert handle.t5a_fwd_dense(C.byref(a), None) == -2          # dtype
    a.dtype = 0
    assert handle.t5a_fwd_dense(C.byref(a), None) == -1          # q is NULL
    a.q = 0x1008
    assert handle.t5a_fwd_dense(C.byref(a), None) == -5          # misaligned
    a.q = 0x1000
    a.q_strides = (C.c_int64 * 3)(0, 0, 63)
    assert handle.t5a_fwd_dense(C.byref(a), None) == -5          # stride
    assert handle.t5a_fwd_dense(None, None) == -1
    a.M = -1
    assert handle.t5a_fwd_dense(C.byref(a), None) == -4
    a.M = 0
    assert handle.t5a_fwd_dense(C.byref(a), None) == 0           # empty problem: nothing to launch
    # one (batch, head) slice of K must stay below 2 GiB: 32-bit byte offsets inside the kernel
    big = lib.T5ADenseArgs()
    big.dtype, big.B, big.H, big.M, big.N, big.D = 0, 1, 1, 8, 1 << 20, 64
    big.q = big.k = big.v = big.o = 0x1000
    for name in ("q_strides", "k_strides", "v_strides", "o_strides"):
        setattr(big, name, (C.c_int64 * 3)(0, 0, 2048))
    assert handle.t5a_fwd_dense(C.byref(big), None) == -4
    assert b"2 GiB" in handle.t5a_last_error()
    s = lib.T5ASparseArgs()
    s.dtype, s.B, s.H, s.L, s.D, s.pattern, s.block_len = 0, 1, 1, 8, 64, 9, 4
    assert handle.t5a_fwd_sparse(C.byref(s), None) == -7
    s.pattern, s.block_len, s.aux = 2, 4, 5
    assert handle.t5a_fwd_sparse(C.byref(s), None) == -7          # more global tokens than the block holds
    k = lib.T5ASplitKArgs()
    k.dtype, k.B, k.H, k.M, k.N, k.D, k.num_splits = 0, 1, 1, 1, 64, 64, 0
    assert handle.t5a_fwd_splitk(C.byref(k), None) == -4
    assert handle.t5a_splitk_workspace_bytes(2, 3, 1, 64, 4) == 2 * 3 * 4 * 1 * 66 * 4


def test_workspace_sizes_and_checks_without_gpu(lib):
    """sizes of the optional buffers, and the checks an entry point makes on them before any launch"""
    handle = lib.load()
    # distance LUTs: (H, 4, qlen) floats with qlen = 4 * (ceil((entries + 6) / 4) ... ) as the kernel lays them out
    for causal, sat in ((0, 91), (1, 113)):           # saturation distances of 32 buckets / max_distance 128
        entries = sat + 96 + (0 if causal else sat) + 96 + 1
        quads = (entries + 6) // 4 + 1
        quads += (4 - quads) % 16          # the four copies start 16 floats apart modulo the 64 LDS banks
        qlen = 4 * quads
        assert handle.t5a_bias_lut_bytes(12, 32, 128, causal) == 12 * 4 * qlen * 4
    assert handle.t5a_bias_lut_bytes(12, 32, 4096, 0) == 0      # too long for the kernel's fetch: not offered
    assert handle.t5a_bias_lut_bytes(0, 32, 128, 0) == 0
    assert handle.t5a_bias_lut_bytes(12, 3, 128, 0) == 0        # bad bucket parameters
    # ... with a sliding window folded in: the image reaches 96 entries past the window when that is wider than the
    # buckets' saturation distance (91 for 32 / 128), and is the plain one's size otherwise
    for window, sat in ((128, 128), (64, 91), (32, 91)):
        quads = (2 * (sat + 96) + 1 + 6) // 4 + 1
        quads += (4 - quads) % 16
        assert handle.t5a_bias_lut_bytes_windowed(12, 32, 128, window) == 12 * 4 * (4 * quads) * 4
    assert handle.t5a_bias_lut_bytes_windowed(12, 32, 128, 256) == 0     # too long for the kernel's fetch
    assert handle.t5a_bias_lut_bytes_windowed(12, 32, 128, 0) == 0
    assert handle.t5a_bias_lut_bytes_windowed(12, 32, 128, 300) == 0     # wider than the windows that go into the LUT
    # launch plan of a packed batch: 64 bytes of counts, 8 lists of 2 * ceil(items / 8) entries of 32 bytes,
    # 16 bytes per item for spilled entries; items = (total_q / 128 + B) * H
    items = (70000 // 128 + 32) * 12
    assert handle.t5a_varlen_workspace_bytes(32, 12, 70000) == 64 + 8 * 2 * ((items + 7) // 8) * 32 + items * 16
    assert handle.t5a_varlen_workspace_bytes(2000, 12, 70000) == 0   # more sequences than the planner holds
    assert handle.t5a_varlen_workspace_bytes(32, 12, 0) == 0
    v = lib.T5AVarlenArgs()
    v.dtype, v.B, v.H, v.D, v.total_q, v.total_k, v.max_seqlen_q, v.max_seqlen_k = 0, 32, 12, 64, 70000, 70000, 4096, 4096
    v.q = v.k = v.v = v.o = v.cu_seqlens_q = v.cu_seqlens_k = 0x1000
    for name in ("q_strides", "k_strides", "v_strides", "o_strides"):
        setattr(v, name, (C.c_int64 * 2)(768, 64))
    v.workspace, v.workspace_bytes = 0x2000, 100
    assert handle.t5a_fwd_varlen(C.byref(v), None) == -8         # workspace too small
    assert b"t5a_varlen_workspace_bytes" in handle.t5a_last_error()
    v.workspace, v.workspace_bytes = 0x2004, 1 << 30
    assert handle.t5a_fwd_varlen(C.byref(v), None) == -5         # workspace misaligned
    d = lib.T5ADenseArgs()
    d.dtype, d.B, d.H, d.M, d.N, d.D = 0, 1, 12, 128, 128, 64
    d.q = d.k = d.v = d.o = 0x1000
    for name in ("q_strides", "k_strides", "v_strides", "o_strides"):
        setattr(d, name, (C.c_int64 * 3)(12 * 128 * 64, 128 * 64, 64))
    d.bias.table, d.bias.table_dtype, d.bias.num_buckets, d.bias.max_distance = 0x3000, 1, 32, 128
    d.bias.stride_bucket, d.bias.stride_head = 12, 1
    d.bias.lut, d.bias.lut_bytes = 0x4000, 64
    assert handle.t5a_fwd_dense(C.byref(d), None) == -8          # LUT buffer too small
    d.bias.lut, d.bias.lut_bytes = 0x4008, 1 << 20
    assert handle.t5a_fwd_dense(C.byref(d), None) == -5          # LUT buffer misaligned


def test_ops_refuse_cpu_tensors():
    from turbot5_amd.ops import flash_attention_with_fusing_bias
    q = torch.zeros(1, 1, 8, 64)
    with pytest.raises(RuntimeError, match="ROCm device"):
        flash_attention_with_fusing_bias(q, q, q, None)


def test_function_signatures_match_the_reference():
    """Names, order and defaults of fused_bias_attention.py:876 and varlen_fused_bias_attn.py:870."""
    from turbot5_amd import ops
    p = list(inspect.signature(ops.flash_attention_with_fusing_bias).parameters.items())[:8]
    assert [(k, v.default) for k, v in p] == [
        ("q", inspect._empty), ("k", inspect._empty), ("v", inspect._empty), ("bias", inspect._empty),
        ("causal", False), ("sm_scale", None), ("NUM_BUCKETS", 32), ("MAX_DISTANCE", 128)]
    p = list(inspect.signature(ops.flash_attention_with_fusing_bias_varlen).parameters.items())[:12]
    assert [k for k, _ in p] == ["q", "k", "v", "bias", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q",
                                 "max_seqlen_k", "causal", "sm_scale", "NUM_BUCKETS", "MAX_DISTANCE"]
    assert [v.default for _, v in p][8:] == [False, None, 32, 128]
    p = list(inspect.signature(ops.flash_attn_v2_fwd).parameters)
    assert p == ["q", "k", "v", "bias", "causal", "sm_scale", "NUM_SPLITS", "BLOCK_M", "BLOCK_N", "num_warps",
                 "num_stages"]


def test_module_surface():
    from turbot5_amd import T5ATTENTION_TYPES, T5Config, T5EncoderModel
    assert {"flash", "local", "block", "transient-global"} <= set(T5ATTENTION_TYPES)
    cfg = T5Config(d_model=64, d_kv=16, d_ff=128, num_layers=2, num_heads=4, vocab_size=50,
                   attention_type="transient-global")
    m = T5EncoderModel(cfg)
    keys = set(m.state_dict())
    p = "encoder.block.0.layer.0.SelfAttention."
    for name in ("q.weight", "k.weight", "v.weight", "o.weight", "relative_attention_bias.weight",
                 "global_relative_attention_bias.weight", "global_input_layer_norm.weight"):
        assert p + name in keys
    assert "encoder.block.1.layer.0.SelfAttention.relative_attention_bias.weight" not in keys
    for name, cls in T5ATTENTION_TYPES.items():
        sig = inspect.signature(cls.forward)
        assert list(sig.parameters)[:3] == ["self", "hidden_states", "mask"]
        assert "position_bias" in sig.parameters and "output_attentions" in sig.parameters
    with pytest.raises(KeyError):
        T5EncoderModel(cfg.copy(attention_type="full"))     # the reference's default is not a registry key either


def test_padding_helpers_on_cpu():
    from turbot5_amd.padding import _get_unpad_data, _upad_input, pad_input
    mask = torch.tensor([[1, 1, 1, 0], [1, 0, 0, 0], [1, 1, 1, 1]])
    idx, cu, mx = _get_unpad_data(mask)
    idx2, cu2, _ = O.unpad_data(mask)
    assert torch.equal(idx, idx2) and torch.equal(cu, cu2) and cu.dtype == torch.int32 and mx == 4
    x = torch.arange(3 * 4 * 2 * 2, dtype=torch.float32).view(3, 4, 2, 2)
    q, k, v, iq, (cq, ck), (mq, mk) = _upad_input(x, x, x, mask, 4, 2)
    assert q.shape == (8, 2, 2) and torch.equal(cq, ck)
    back = pad_input(q, iq, 3, 4)
    assert torch.equal(back[mask.bool()], x[mask.bool()])
    assert torch.equal(back[~mask.bool()], torch.zeros_like(back[~mask.bool()]))


def test_packed_workload_lengths_fixture():
    import json
    fx = json.load(open(os.path.join(ROOT, "tests", "golden", "c3_lengths.json")))
    lens = torch.randint(128, 4097, (32,), generator=torch.Generator().manual_seed(1)).tolist()
    assert fx["lengths"] == lens and fx["total"] == sum(lens)
    import bench
    assert bench.c3_lengths() == lens


def test_mask_info_is_not_inherited_by_another_tensor():
    """The per-mask cache is keyed by address and version, which a new tensor can share with a freed one: an
    entry only counts while the tensor it was made for is alive and is the one asked about."""
    import gc
    import weakref
    from turbot5_amd import attentions as A
    A._MASK_INFO.clear()
    m = torch.tensor([[1, 1, 1, 0], [1, 0, 0, 0]])
    all_ones, unpad = A._mask_info(m)
    assert not all_ones and unpad[0] == "lens" and unpad[1][0].tolist() == [3, 1]
    assert A._mask_info(m)[1] is unpad                      # same tensor: served from the cache
    m2 = torch.tensor([[1, 1, 0, 0], [1, 1, 1, 1]])
    key2 = (m2.data_ptr(), m2._version, tuple(m2.shape), str(m2.device), m2.dtype)
    A._MASK_INFO[key2] = (weakref.ref(m), all_ones, unpad)   # what address reuse would leave behind
    assert A._mask_info(m2)[1][1][0].tolist() == [2, 4]
    ref = A._MASK_INFO[(m.data_ptr(), m._version, tuple(m.shape), str(m.device), m.dtype)][0]
    del m
    gc.collect()
    assert ref() is None


def test_sequence_length_arguments_are_checked_without_gpu(lib):
    """seq_starts belongs to the windowed patterns and needs seq_lens; the checks come before any launch"""
    handle = lib.load()
    s = lib.T5ASparseArgs()
    s.dtype, s.B, s.H, s.L, s.D, s.pattern, s.block_len, s.aux = 0, 1, 1, 256, 64, 2, 64, 16    # block pattern
    s.q = s.k = s.v = s.o = 0x1000
    for name in ("q_strides", "k_strides", "v_strides", "o_strides"):
        setattr(s, name, (C.c_int64 * 3)(256 * 64, 256 * 64, 64))
    s.seq_lens, s.seq_starts = 0x3000, 0x3100
    assert handle.t5a_fwd_sparse(C.byref(s), None) == -7           # first rows: windowed patterns only
    assert b"seq_starts" in handle.t5a_last_error()
    s.pattern, s.aux, s.seq_lens = 1, 0, None
    assert handle.t5a_fwd_sparse(C.byref(s), None) == -7           # first rows without lengths
    assert b"seq_starts" in handle.t5a_last_error()
    r = lib.T5ARmsNormArgs()
    r.x, r.weight, r.y = 0x1000, 0x2000, 0x4000
    r.x_strides = (C.c_int64 * 2)(0, 64)
    r.batches, r.rows_per_batch, r.dim, r.group = 1, 8, 64, 1
    r.x_dtype, r.weight_dtype, r.eps = 0, 0, 1e-6
    r.seq_lens = 0x3000
    r.residual, r.sum_out, r.residual_row_stride = 0x5000, 0x6000, 64
    assert handle.t5a_rmsnorm(C.byref(r), None) == -4          # lengths and a residual do not go together
    assert b"seq_lens" in handle.t5a_last_error()
    r.seq_lens = None
    r.seq_starts = 0x3100
    r.residual = None
    assert handle.t5a_rmsnorm(C.byref(r), None) == -4          # first rows without lengths
    r.seq_starts, r.residual = None, 0x5000
    r.group, r.rows_per_batch = 2, 8
    assert handle.t5a_rmsnorm(C.byref(r), None) == -4          # a residual needs group == 1
    r.group, r.sum_out = 1, 0x1000
    assert handle.t5a_rmsnorm(C.byref(r), None) == -5          # sum_out must not be x


def test_packed_batch_layout_and_mask_kinds():
    """Host logic either side of the packed kernel: which masks run in place, which are right padded (the
    windowed patterns' case), and the packed layout a whole stack runs on."""
    from turbot5_amd import attentions as A
    A._MASK_INFO.clear()
    ones = torch.ones(2, 5)
    assert A._mask_info(ones) == (True, None) and A.packed_batch(ones) is None
    right = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1], [0, 0, 0, 0, 0]])
    all_ones, (kind, (lens, cu), extra) = A._mask_info(right)
    assert not all_ones and kind == "lens" and extra["right_padded"]
    assert lens.tolist() == [3, 5, 0] and cu.tolist() == [0, 5, 10, 15]
    pb = A.packed_batch(right)
    assert pb.indices.tolist() == [0, 1, 2, 5, 6, 7, 8, 9] and pb.cu_seqlens.tolist() == [0, 3, 8, 8]
    assert (pb.batch, pb.length, pb.max_len) == (3, 5, 5) and A.packed_batch(right) is pb
    left = torch.tensor([[0, 0, 1, 1, 1], [1, 1, 1, 1, 0]])
    _, (kind, (lens, cu), extra) = A._mask_info(left)
    assert kind == "lens" and not extra["right_padded"] and lens.tolist() == [3, 4] and cu.tolist() == [2, 5, 10]
    holes = torch.tensor([[1, 0, 1, 1, 0], [1, 1, 1, 1, 1]])
    _, (kind, (indices, cu, max_len), _) = A._mask_info(holes)
    assert kind == "packed" and indices.tolist() == [0, 2, 3, 5, 6, 7, 8, 9] and cu.tolist() == [0, 3, 8]
    assert A.packed_batch(holes).indices is indices


@pytest.mark.parametrize("cus", [64, 104, 256, 304])
def test_sparse_launch_plans_cover_every_item(lib, cus):
    """The launch plan of the sparse patterns over a grid of shapes and device sizes: the runs cover the
    (batch, head, q tile) list exactly, and when the global rows of the block pattern travel in the same launch,
    their key splits cover the keys exactly, with at least one split per (batch, head) and never more than the
    workspace was sized for.  Shapes with many (batch, head) pairs end with ONE split per pair: still a split item
    of its own behind the runs (the kernel tells the folded launch by its number of block items)."""
    L_ = lib.load()
    out = (C.c_int32 * 6)()
    seen_single_split = False
    for B in (1, 2, 4, 8, 16, 33):
        for H in (1, 8, 12, 16):
            for L in (128, 500, 1024, 2048, 4096, 16384):
                for Bl, G in ((128, 64), (64, 32), (256, 128), (100, 20), (512, 0)):
                    if G > Bl:
                        continue
                    for run_len in (0, 1, 5, 16):
                        rc = L_.t5a_sparse_launch_plan(lib.PATTERN_BLOCK, lib.T5A_BF16, B, H, L, 64, Bl, G, 1, cus, run_len, out)
                        assert rc == 0, (B, H, L, Bl, G, run_len, L_.t5a_last_error())
                        rl, items, block_items, nsplit, split_rows, tps = list(out)
                        entries = tps * B * H
                        runs = block_items if block_items > 0 else items
                        assert 1 <= rl <= 16 and runs * rl >= entries > (runs - 1) * rl, (B, H, L, Bl, G, run_len, list(out))
                        if run_len:
                            assert rl == run_len or L < Bl
                        if block_items > 0:
                            assert items == block_items + nsplit * B * H and nsplit >= 1
                            assert nsplit * split_rows >= L > (nsplit - 1) * split_rows and split_rows % 64 == 0
                            ws = L_.t5a_sparse_workspace_bytes(lib.PATTERN_BLOCK, B, H, L, 64, Bl, G)
                            assert B * H * nsplit * min(G, L) * (64 + 2) * 4 <= ws
                            seen_single_split |= nsplit == 1
                        else:
                            assert nsplit == 0
    assert seen_single_split or cus > 256
    # the local pattern: runs only; fp32 and other head dims: one q tile per item
    for dtype, D, want_runs in ((lib.T5A_BF16, 64, True), (lib.T5A_F32, 64, False), (lib.T5A_BF16, 32, False)):
        assert L_.t5a_sparse_launch_plan(lib.PATTERN_LOCAL, dtype, 1, 12, 16384, D, 128, 0, 0, cus, 0, out) == 0
        rl, items, block_items, nsplit, split_rows, tps = list(out)
        assert tps == 128 and block_items == 0 and items * rl >= 128 * 12 > (items - 1) * rl
        assert (rl > 1) == (want_runs and 2 * cus < 128 * 12)
    assert L_.t5a_sparse_launch_plan(lib.PATTERN_BLOCK, lib.T5A_BF16, 1, 1, 128, 64, 128, 64, 1, cus, 17, out) < 0
    assert L_.t5a_sparse_launch_plan(9, lib.T5A_BF16, 1, 1, 128, 64, 128, 64, 1, cus, 0, out) < 0
