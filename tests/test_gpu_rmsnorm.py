"""GPU parity of the fused RMS norm / side-token producer against the CPU oracle (through the C ABI)."""
import pytest
import torch

from oracle import t5_basic as O
from oracle.t5_model import tglobal_side_inputs

pytestmark = pytest.mark.gpu

DT = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}


@pytest.mark.parametrize("xdt,wdt", [("bf16", "bf16"), ("f32", "f32"), ("f32", "bf16"), ("bf16", "f32"), ("f16", "f16")])
@pytest.mark.parametrize("shape", [(2, 100, 768), (3, 7, 512), (1, 16384, 768), (5, 4096), (2, 9, 64), (4, 33, 4096)])
def test_rms_norm_matches_the_oracle(gpu_device, xdt, wdt, shape):
    from turbot5_amd.ops import rms_norm
    g = torch.Generator().manual_seed(sum(shape) + len(xdt) * 7 + len(wdt))
    x = (2.0 * torch.randn(*shape, generator=g)).to(DT[xdt])
    w = (1.0 + 0.2 * torch.randn(shape[-1], generator=g)).to(DT[wdt])
    want = O.rms_norm(x, w, 1e-6)
    got = rms_norm(x.to(gpu_device), w.to(gpu_device), 1e-6)
    assert got.dtype == want.dtype and got.shape == want.shape
    diff = (got.float().cpu() - want.float()).abs()
    if want.dtype == torch.float32:
        assert (diff <= 2e-6 + 1e-5 * want.float().abs()).all()
    else:
        # two roundings (scaled value, then product): a last-bit difference of the fp32 scale can move the
        # result by up to two units in the last place; it almost never does
        ulp = 2.0 ** -7 if want.dtype == torch.bfloat16 else 2.0 ** -10
        assert (diff <= 2 * ulp * want.float().abs() + 1e-6).all()
        assert (diff == 0).float().mean().item() > 0.98


def test_rms_norm_strided_rows_and_closed_form(gpu_device):
    from turbot5_amd.ops import rms_norm
    big = torch.randn(4, 50, 1024, generator=torch.Generator().manual_seed(3))
    x = big[:, :, 256:768]                                           # row stride 1024, 512 columns
    w = torch.ones(512)
    got = rms_norm(x.to(gpu_device)[:, :, :], w.to(gpu_device)).cpu()
    assert torch.allclose(got.pow(2).mean(-1), torch.ones(4, 50), atol=1e-4)   # unit RMS by definition
    assert torch.allclose(got, O.rms_norm(x, w), atol=1e-5, rtol=1e-5)
    const = torch.full((3, 64), 5.0)                                 # constant row -> weight itself
    w2 = torch.linspace(-1, 1, 64)
    assert torch.allclose(rms_norm(const.to(gpu_device), w2.to(gpu_device), 0.0).cpu(), w2.expand(3, 64), atol=1e-6)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("L,gbs", [(512, 16), (100, 16), (37, 8), (16, 16), (15, 16), (2048, 1), (130, 64)])
def test_side_token_producer_matches_the_oracle(gpu_device, dtype, L, gbs):
    """Block sums + norm in one kernel, against the one-hot einsum + norm of the oracle; L % gbs != 0
    exercises the orphan tokens that join the last full block."""
    from turbot5_amd.ops import rms_norm
    B, d = 3, 256
    g = torch.Generator().manual_seed(L * 31 + gbs)
    hidden = torch.randn(B, L, d, generator=g).to(DT[dtype])
    w = (1.0 + 0.1 * torch.randn(d, generator=g)).to(DT[dtype])
    want = tglobal_side_inputs(hidden, gbs, w, 1e-6)
    got = rms_norm(hidden.to(gpu_device), w.to(gpu_device), 1e-6, group=gbs)
    assert got.shape == want.shape == (B, L // gbs, d)
    if want.numel():
        tol = 1e-5 if dtype == "f32" else 2e-2                        # bf16: the einsum's accumulation order is free
        assert (got.float().cpu() - want.float()).abs().max().item() <= tol * max(1.0, want.float().abs().max().item())


def test_layer_norm_module_uses_the_kernel(gpu_device):
    from turbot5_amd.attentions import T5LayerNorm
    torch.manual_seed(0)
    m = T5LayerNorm(768).to(gpu_device).to(torch.bfloat16)
    x = torch.randn(2, 300, 768).to(torch.bfloat16)
    want = O.rms_norm(x, m.weight.detach().cpu(), m.eps)
    got = m(x.to(gpu_device))
    assert got.dtype == torch.bfloat16
    assert (got.float().cpu() - want.float()).abs().max().item() <= 2.0 ** -6


@pytest.mark.parametrize("xdt,wdt", [("bf16", "bf16"), ("f32", "f32"), ("f16", "f16"), ("f32", "bf16")])
@pytest.mark.parametrize("shape", [(2, 100, 768), (1, 4096, 768), (3, 7, 512), (2, 9, 64), (2, 33, 4096), (1, 5, 2048)])
def test_add_then_norm_in_one_kernel(gpu_device, xdt, wdt, shape):
    """x + residual (rounded to x's type, exactly torch's add) and the norm of that sum; covers rows held
    in registers (two and four chunks per lane) and the two-pass form (4096 columns)."""
    from turbot5_amd.ops import rms_norm
    g = torch.Generator().manual_seed(sum(shape) + len(xdt))
    x = (2.0 * torch.randn(*shape, generator=g)).to(DT[xdt])
    r = (1.5 * torch.randn(*shape, generator=g)).to(DT[xdt])
    w = (1.0 + 0.2 * torch.randn(shape[-1], generator=g)).to(DT[wdt])
    total, got = rms_norm(x.to(gpu_device), w.to(gpu_device), 1e-6, residual=r.to(gpu_device))
    assert torch.equal(total.cpu(), x + r)                      # one correctly rounded add: bit-exact
    want = O.rms_norm(x + r, w, 1e-6)
    assert got.dtype == want.dtype and got.shape == want.shape and total.dtype == x.dtype
    plain = rms_norm((x + r).to(gpu_device), w.to(gpu_device), 1e-6)
    assert torch.equal(got, plain)                              # same arithmetic as the norm alone on the sum
    diff = (got.float().cpu() - want.float()).abs()
    ulp = {torch.float32: 1e-5, torch.bfloat16: 2.0 ** -6, torch.float16: 2.0 ** -9}[want.dtype]
    assert (diff <= ulp * want.float().abs() + 2e-6).all()


def test_add_norm_rejects_bad_arguments(gpu_device):
    from turbot5_amd.ops import rms_norm
    x = torch.randn(2, 8, 64, device=gpu_device)
    w = torch.ones(64, device=gpu_device)
    with pytest.raises(ValueError):
        rms_norm(x, w, residual=x[:, :4])
    with pytest.raises(ValueError):
        rms_norm(x, w, group=2, residual=x)
    with pytest.raises(ValueError):
        rms_norm(x, w, residual=x.half())


def test_layer_norm_add_norm_and_stack_equivalence(gpu_device):
    """The stack hands each sub-layer's update to the next norm; block.forward adds it itself: same numbers."""
    from turbot5_amd import T5Config, T5EncoderModel
    torch.manual_seed(3)
    cfg = T5Config(vocab_size=100, d_model=128, d_kv=64, d_ff=256, num_layers=2, num_heads=2, dropout_rate=0.0,
                   attention_type="flash")
    m = T5EncoderModel(cfg).eval().to(gpu_device).to(torch.bfloat16)
    ids = torch.randint(0, 100, (2, 70), device=gpu_device)
    with torch.no_grad():
        got = m(ids)
        h = m.shared(ids)
        bias = None
        for blk in m.encoder.block:
            h, _, bias = blk(h, position_bias=bias)
        want = m.encoder.final_layer_norm(h)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("L,gbs,lens", [(512, 16, [512, 300, 17, 0]), (100, 16, [99, 16, 15, 64]), (64, 8, [64, 63, 9, 1])])
def test_side_token_producer_with_sequence_lengths(gpu_device, dtype, L, gbs, lens):
    """Right-padded batch: a sequence of n tokens has n // gbs side tokens (its last tokens join the last
    full block, padding is left out), the remaining output rows are zero -- the oracle's mask path."""
    from turbot5_amd.ops import rms_norm
    B, d = len(lens), 256
    g = torch.Generator().manual_seed(L * 13 + gbs)
    hidden = torch.randn(B, L, d, generator=g).to(DT[dtype])
    w = (1.0 + 0.1 * torch.randn(d, generator=g)).to(DT[dtype])
    mask = (torch.arange(L)[None, :] < torch.tensor(lens)[:, None]).float()
    want = tglobal_side_inputs(hidden, gbs, w, 1e-6, mask)
    got = rms_norm(hidden.to(gpu_device), w.to(gpu_device), 1e-6, group=gbs,
                   seq_lens=torch.tensor(lens, dtype=torch.int32, device=gpu_device))
    assert got.shape == want.shape == (B, L // gbs, d)
    tol = 1e-5 if dtype == "f32" else 2e-2
    assert (got.float().cpu() - want.float()).abs().max().item() <= tol * max(1.0, want.float().abs().max().item())
    for b, n in enumerate(lens):
        assert (got[b, n // gbs:] == 0).all()
    # one side token per token (group 1): every valid row normalised by itself, padding rows zero
    tl = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
    one = rms_norm(hidden.to(gpu_device), w.to(gpu_device), 1e-6, group=1, seq_lens=tl)
    want1 = tglobal_side_inputs(hidden, 1, w, 1e-6, mask)
    assert one.shape == want1.shape == (B, L, d)
    assert (one.float().cpu() - want1.float()).abs().max().item() <= tol * max(1.0, want1.float().abs().max().item())
    with pytest.raises(ValueError):
        rms_norm(hidden.to(gpu_device), w.to(gpu_device), 1e-6, group=1, seq_lens=tl, residual=hidden.to(gpu_device))


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("L,gbs", [(512, 16), (100, 16), (64, 8), (777, 32)])
def test_side_token_producer_with_masks_of_any_shape(gpu_device, dtype, L, gbs):
    """key_bits and group_counts: a side token sums the valid tokens of its block, the last one every valid token
    from its block on, rows past the count are zero -- the oracle's block ids and aggregates for any mask"""
    from turbot5_amd.ops import pack_key_bits, rms_norm, side_token_counts
    B, d = 5, 256
    g = torch.Generator().manual_seed(L * 7 + gbs)
    hidden = torch.randn(B, L, d, generator=g).to(DT[dtype])
    w = (1.0 + 0.1 * torch.randn(d, generator=g)).to(DT[dtype])
    mask = torch.ones(B, L)
    mask[0] = (torch.rand(L, generator=g) > 0.3).float()
    mask[1, : L // 3] = 0
    mask[2, L // 5: L // 2] = 0
    mask[2, -(gbs + 3):] = 0
    mask[3, gbs - 1::gbs] = 0          # no block END is valid: no side token
    want = tglobal_side_inputs(hidden, gbs, w, 1e-6, mask)
    dmask = mask.to(gpu_device)
    counts = side_token_counts(dmask, gbs)
    got = rms_norm(hidden.to(gpu_device), w.to(gpu_device), 1e-6, group=gbs, key_bits=pack_key_bits(dmask, gbs),
                   group_counts=counts)
    assert got.shape == want.shape == (B, L // gbs, d)
    tol = 1e-5 if dtype == "f32" else 2e-2
    assert (got.float().cpu() - want.float()).abs().max().item() <= tol * max(1.0, want.float().abs().max().item())
    assert (got[3] == 0).all() and counts[3].item() == 0
    for b in range(B):
        assert (got[b, counts[b].item():] == 0).all()
    with pytest.raises(ValueError):
        rms_norm(hidden.to(gpu_device), w.to(gpu_device), 1e-6, group=gbs, key_bits=pack_key_bits(dmask, gbs))
