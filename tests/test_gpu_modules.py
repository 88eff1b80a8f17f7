"""GPU parity of the attention modules and the layer stack against the CPU oracle model
(same state dict on both sides)."""
import pytest
import torch

from oracle import t5_model as OM

pytestmark = pytest.mark.gpu


def make(cfg_kwargs, model="encoder", seed=0):
    from turbot5_amd import T5Config, T5EncoderModel, T5Model
    torch.manual_seed(seed)
    cfg = T5Config(**cfg_kwargs)
    m = (T5EncoderModel if model == "encoder" else T5Model)(cfg).eval()
    with torch.no_grad():   # make the bias table and norms matter
        for name, p in m.named_parameters():
            if "relative_attention_bias" in name:
                p.copy_(torch.randn_like(p))
            if "layer_norm" in name:
                p.copy_(1.0 + 0.1 * torch.randn_like(p))
    sd = {k: v.detach().clone() for k, v in m.state_dict().items()}
    return cfg, m, sd


SMALL = dict(vocab_size=200, d_model=128, d_kv=64, d_ff=256, num_layers=2, num_heads=2, dropout_rate=0.0)


@pytest.mark.parametrize("attention_type,L,extra", [
    ("flash", 200, {}),
    ("local", 256, dict(sliding_window=64)),
    ("local", 40, dict(sliding_window=64)),
    ("block", 256, dict(sliding_window=64, global_block_size=16)),
    ("block", 40, dict(sliding_window=64, global_block_size=16)),
    ("transient-global", 256, dict(sliding_window=64, global_block_size=8)),
    ("transient-global", 200, dict(sliding_window=64, global_block_size=16)),   # trailing tokens join the last block
])
def test_encoder_types_fp32(gpu_device, attention_type, L, extra):
    cfg, m, sd = make(dict(SMALL, attention_type=attention_type, **extra))
    ids = torch.randint(0, 200, (2, L), generator=torch.Generator().manual_seed(1))
    want = OM.encoder_forward(sd, cfg, ids, None, attention_type)
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device))                              # no mask
        got2 = m(ids.to(gpu_device), torch.ones(2, L, device=gpu_device))   # explicit all-ones mask
    assert (got.cpu() - want).abs().max().item() <= 2e-3
    assert torch.equal(got, got2)


def test_attention_module_output_tuple(gpu_device):
    from turbot5_amd import T5ATTENTION_TYPES, T5Config
    cfg = T5Config(**dict(SMALL, sliding_window=32, global_block_size=8))
    x = torch.randn(2, 96, 128, device=gpu_device)
    for name, cls in T5ATTENTION_TYPES.items():
        mod = cls(cfg, has_relative_attention_bias=True).to(gpu_device).eval()
        with torch.no_grad():
            out = mod(x, mask=torch.ones(2, 96, device=gpu_device))
        assert len(out) == 3 and out[0].shape == (2, 96, 128) and out[1] is None
        assert out[2] is mod.relative_attention_bias.weight      # the table, handed on to later layers
        later = cls(cfg, has_relative_attention_bias=False).to(gpu_device).eval()
        with torch.no_grad():
            out2 = later(x, position_bias=out[2])
        assert out2[0].shape == (2, 96, 128)
    mask = torch.ones(2, 96, device=gpu_device)
    mask[1, 50:] = 0
    mask[0, :3] = 0
    with torch.no_grad():                            # left padding: every pattern
        for name in ("local", "block", "transient-global"):
            out = T5ATTENTION_TYPES[name](cfg, has_relative_attention_bias=True).to(gpu_device).eval()(x, mask=mask)
            assert torch.isfinite(out[0][mask.bool()]).all()
        mask[1, 20:30] = 0                           # holes: validity bit sets
        for name in ("local", "block", "transient-global"):
            out = T5ATTENTION_TYPES[name](cfg, has_relative_attention_bias=True).to(gpu_device).eval()(x, mask=mask)
            assert torch.isfinite(out[0][mask.bool()]).all()


def test_output_attentions_gives_a_fourth_element_none(gpu_device):
    """The reference's fused modules accept output_attentions=True and return None as the weights
    (attentions.py:483, :519-520, :647, :860, :1063); so do these, with the other three elements unchanged."""
    from turbot5_amd import T5ATTENTION_TYPES, T5Config
    cfg = T5Config(**dict(SMALL, sliding_window=32, global_block_size=8))
    x = torch.randn(2, 96, 128, device=gpu_device)
    for name, cls in T5ATTENTION_TYPES.items():
        mod = cls(cfg, has_relative_attention_bias=True).to(gpu_device).eval()
        with torch.no_grad():
            plain = mod(x)
            out = mod(x, output_attentions=True)
        assert len(plain) == 3 and len(out) == 4 and out[3] is None, name
        assert torch.equal(out[0], plain[0]) and out[1] is None and out[2] is plain[2]


@pytest.mark.parametrize("activations", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sigma", [8.0, 18.0])
@pytest.mark.parametrize("kind", ["flash", "local", "block", "transient-global"])
def test_modules_hold_2e2_at_unscaled_t5_score_magnitudes(gpu_device, kind, sigma, activations):
    """T5 does not scale its scores, so trained checkpoints have scores of deviation 8 and more.  With the DEFAULT
    config the modules fold log2(e) into the query projection (the rows are rounded to bf16 once, the kernel
    applies no factor), and the attention output -- taken at the input of the output projection -- stays within
    2e-2 of fp32 'basic' math on the rows, keys and values that the kernel was given: the rows divided by log2(e)
    again, which costs a relative 2^-24.  fp32 activations with bf16 attention, and bf16 throughout."""
    from turbot5_amd import T5ATTENTION_TYPES, T5Config, ops
    from oracle import t5_basic as O
    H, D, L, B, Bl, aux = 2, 64, 512, 2, 128, 16
    cfg = T5Config(vocab_size=32, d_model=H * D, d_kv=D, d_ff=2 * H * D, num_layers=1, num_heads=H, dropout_rate=0.0,
                   attention_type=kind, sliding_window=Bl, global_block_size=aux,
                   attention_dtype=torch.bfloat16 if activations == torch.float32 else None)
    assert cfg.attention_exact_scores is None
    g = torch.Generator().manual_seed(int(sigma) * 7 + len(kind))
    mod = T5ATTENTION_TYPES[kind](cfg, has_relative_attention_bias=True).eval()
    with torch.no_grad():
        # q.k over head_dim 64 has deviation sigma when the rows and keys have variance sigma / 8
        std = (sigma / 8.0) ** 0.5
        for name, prm in mod.named_parameters():
            if "relative_attention_bias" in name:
                prm.copy_(torch.randn(prm.shape, generator=g))
            elif name.startswith(("q.", "k.")):
                prm.copy_(torch.randn(prm.shape, generator=g) * std * prm.shape[1] ** -0.5)
            elif name.startswith(("v.", "o.")):
                prm.copy_(torch.randn(prm.shape, generator=g) * prm.shape[1] ** -0.5)
    mod = mod.to(gpu_device).to(activations)
    hidden = torch.randn(B, L, H * D, generator=g).to(gpu_device).to(activations)
    seen = {}
    mod.o.register_forward_pre_hook(lambda m, args: seen.__setitem__("attn", args[0].detach()))
    calls = []
    real = ops.prescaled_query
    try:
        ops.prescaled_query = lambda *a, **k: calls.append(real(*a, **k)) or calls[-1]
        with torch.no_grad():
            mod(hidden)
    finally:
        ops.prescaled_query = real
    assert len(calls) == 1 and calls[0].dtype == torch.bfloat16   # the default config took the folded projection

    def heads(x):
        return x.float().cpu().view(B, -1, H, D).transpose(1, 2)
    with torch.no_grad():
        q = heads(calls[0]) / ops.LOG2E
        k, v = (heads(p(hidden).to(torch.bfloat16)) for p in (mod.k, mod.v))
        table = mod.relative_attention_bias.weight.float().cpu()
        if kind == "flash":
            want = O.dense_attention(q, k, v, table, False, 1.0)
        elif kind == "local":
            want = O.local_attention_blocked(q, k, v, table, Bl)
        elif kind == "block":
            want = O.block_attention_blocked(q, k, v, table, Bl, aux)
        else:
            side = mod.side_inputs(hidden)
            sk, sv = (heads(p(side).to(torch.bfloat16)) for p in (mod.k, mod.v))
            want = O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, aux)
    # the scores really are that large
    s = torch.einsum("bhid,bhjd->bhij", q, k)
    assert 0.8 * sigma <= s.std().item() <= 1.25 * sigma
    got = heads(seen["attn"])
    err = (got - want).abs().max().item()
    assert err <= 2e-2, f"{kind} sigma {sigma}: max-abs {err}"


def test_flash_encoder_with_padding(gpu_device):
    """A right-padded batch runs in place through the packed kernel with per-sequence lengths."""
    cfg, m, sd = make(dict(SMALL, attention_type="flash"))
    ids = torch.randint(0, 200, (3, 150), generator=torch.Generator().manual_seed(2))
    mask = torch.ones(3, 150)
    mask[0, 100:] = 0
    mask[2, 1:] = 0
    want = OM.encoder_forward(sd, cfg, ids, mask)
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device), mask.to(gpu_device)).cpu()
    valid = mask.bool()
    assert (got[valid] - want[valid]).abs().max().item() <= 2e-3


def test_flash_encoder_with_left_padding_and_holes(gpu_device):
    """A mask that is not a run of ones followed by zeros cannot run in place: it takes the gather /
    packed kernel / scatter route (the reference's only route, attentions.py:492-511).  As in the
    reference, positions are counted over the VALID tokens of a sequence (padding.py:113-150 packs them
    before the kernel numbers them, varlen_fused_bias_attn.py:254, :303), so each sequence equals the
    oracle run on its valid tokens alone."""
    cfg, m, sd = make(dict(SMALL, attention_type="flash"))
    ids = torch.randint(0, 200, (3, 140), generator=torch.Generator().manual_seed(5))
    mask = torch.ones(3, 140)
    mask[0, :30] = 0                 # left padding
    mask[1, 50:60] = 0               # a hole
    mask[2, 100:] = 0                # right padding in the same batch
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device), mask.to(gpu_device)).cpu()
    for b in range(3):
        valid = mask[b].bool()
        want = OM.encoder_forward(sd, cfg, ids[b][valid][None])[0]
        assert (got[b][valid] - want).abs().max().item() <= 2e-3


def test_flash_encoder_with_padding_on_either_side_runs_in_place(gpu_device):
    """Rows that are one run of valid tokens (left padding, right padding, both, none, or no token at all) run
    in place with a start row and a length per sequence; each sequence equals the oracle on its valid tokens
    and the padded positions of the attention output are zero."""
    from turbot5_amd import attentions as A
    cfg, m, sd = make(dict(SMALL, attention_type="flash"))
    ids = torch.randint(0, 200, (5, 150), generator=torch.Generator().manual_seed(6))
    mask = torch.ones(5, 150)
    mask[0, :40] = 0                 # left padding
    mask[1, 90:] = 0                 # right padding
    mask[2, :10] = 0
    mask[2, 130:] = 0                # both
    mask[4, :] = 0                   # nothing valid
    dmask = mask.to(gpu_device)
    assert A._mask_info(dmask)[1][0] == "lens"
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device), dmask).cpu()
    for b in range(4):
        valid = mask[b].bool()
        want = OM.encoder_forward(sd, cfg, ids[b][valid][None])[0]
        assert (got[b][valid] - want).abs().max().item() <= 2e-3, b
    assert torch.isfinite(got).all()


def test_bf16_attention_inside_fp32_model(gpu_device):
    cfg, m, sd = make(dict(SMALL, attention_type="flash", attention_dtype=torch.bfloat16))
    ids = torch.randint(0, 200, (2, 300), generator=torch.Generator().manual_seed(3))
    want = OM.encoder_forward(sd, cfg, ids)
    with torch.no_grad():
        got = m.to(gpu_device)(ids.to(gpu_device)).cpu()
    assert got.dtype == torch.float32
    assert (got - want).abs().max().item() <= 6e-2     # two layers of bf16 attention inside fp32 activations


def test_config1_t5_small_encoder(gpu_device):
    """Baseline configuration 1: T5-small random init (seed 0), batch 4 x 512 ids, all-ones mask, fp32."""
    cfg, m, sd = make(dict(vocab_size=32128, d_model=512, d_kv=64, d_ff=2048, num_layers=6, num_heads=8,
                           dropout_rate=0.0, attention_type="flash"), seed=0)
    ids = torch.randint(0, 32128, (4, 512), generator=torch.Generator().manual_seed(0))
    want = OM.encoder_forward(sd, cfg, ids)
    with torch.no_grad():
        got = m.to(gpu_device)(ids.to(gpu_device), torch.ones(4, 512, device=gpu_device)).cpu()
    err = (got - want).abs().max().item()
    assert err <= 2e-3, err     # six fp32 layers end to end; each attention op is held to 1e-4 in test_gpu_dense.py


def test_encoder_decoder_and_greedy_decode(gpu_device):
    cfg, m, sd = make(dict(SMALL, attention_type="flash", num_decoder_layers=2), model="t5")
    ids = torch.randint(0, 200, (2, 600), generator=torch.Generator().manual_seed(4))
    dec = torch.randint(0, 200, (2, 130), generator=torch.Generator().manual_seed(5))
    mem = OM.encoder_forward(sd, cfg, ids)
    want = OM.lm_logits(sd, cfg, OM.decoder_forward(sd, cfg, dec, mem))
    m = m.to(gpu_device)
    with torch.no_grad():
        logits, enc, _ = m(ids.to(gpu_device), dec.to(gpu_device))
    assert (enc.cpu() - mem).abs().max().item() <= 2e-3
    assert (logits.cpu() - want).abs().max().item() <= 5e-3
    # incremental decoding with the KV cache and the split-K cross-attention reproduces the full pass
    toks = m.greedy_decode(ids.to(gpu_device), max_new_tokens=12).cpu()
    seq = torch.zeros(2, 1, dtype=torch.long)
    for _ in range(12):
        lg = OM.lm_logits(sd, cfg, OM.decoder_forward(sd, cfg, seq, mem))
        seq = torch.cat([seq, lg[:, -1].argmax(-1, keepdim=True)], dim=1)
    assert torch.equal(toks, seq[:, 1:])


def test_cross_attention_with_padded_memory(gpu_device):
    cfg, m, sd = make(dict(SMALL, attention_type="flash", num_decoder_layers=1), model="t5")
    ids = torch.randint(0, 200, (2, 90), generator=torch.Generator().manual_seed(6))
    mask = torch.ones(2, 90)
    mask[1, 60:] = 0
    dec = torch.randint(0, 200, (2, 7), generator=torch.Generator().manual_seed(7))
    mem = OM.encoder_forward(sd, cfg, ids, mask)
    want = OM.lm_logits(sd, cfg, OM.decoder_forward(sd, cfg, dec, mem, mask))
    m = m.to(gpu_device)
    with torch.no_grad():
        logits, _, _ = m(ids.to(gpu_device), dec.to(gpu_device), attention_mask=mask.to(gpu_device))
    assert (logits.cpu() - want).abs().max().item() <= 5e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_relu_epilogue_path_equals_separate_relu(gpu_device, dtype):
    """Inference folds ReLU into wi's GEMM; the result must equal linear -> relu -> linear."""
    from turbot5_amd import T5Config
    from turbot5_amd.modeling import T5DenseActDense
    torch.manual_seed(5)
    ff = T5DenseActDense(T5Config(**SMALL)).to(gpu_device).to(dtype).eval()
    assert "_zero_bias" not in ff.state_dict()
    x = torch.randn(3, 70, 128, device=gpu_device).to(dtype)
    with torch.no_grad():
        got = ff(x)
        want = ff.wo(torch.relu(ff.wi(x)))
    assert got.shape == want.shape == (3, 70, 128)
    assert (got.float() - want.float()).abs().max().item() <= 2e-2 * want.float().abs().max().item()
    x.requires_grad_(True)      # with gradients wanted the layer takes the plain path
    ff(x).sum().backward()
    assert x.grad is not None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gated_gelu_epilogue_path(gpu_device, dtype):
    """'gated-gelu' (T5 v1.1): tanh-GELU in the epilogue of wi_0.  fp32 agrees to rounding; in bf16 the
    epilogue rounds once (after the activation) where the separate kernels round twice."""
    from turbot5_amd import T5Config
    from turbot5_amd.modeling import T5DenseGatedActDense
    torch.manual_seed(6)
    cfg = T5Config(**dict(SMALL, feed_forward_proj="gated-gelu"))
    assert cfg.dense_act_fn == "gelu_new" and cfg.is_gated_act
    ff = T5DenseGatedActDense(cfg).to(gpu_device).to(dtype).eval()
    assert "_zero_bias" not in ff.state_dict()
    x = torch.randn(3, 70, 128, device=gpu_device).to(dtype)
    with torch.no_grad():
        got = ff(x)
        want64 = (torch.nn.functional.gelu(x.double() @ ff.wi_0.weight.double().t(), approximate="tanh")
                  * (x.double() @ ff.wi_1.weight.double().t())) @ ff.wo.weight.double().t()
        plain = ff.wo(ff.act(ff.wi_0(x)) * ff.wi_1(x))
    assert got.shape == (3, 70, 128)
    scale = want64.abs().max().item()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert (got.double() - want64).abs().max().item() <= tol * scale
    # no worse than the separate kernels against exact arithmetic (a little slack for the different rounding)
    assert (got.double() - want64).abs().max().item() <= 1.5 * (plain.double() - want64).abs().max().item() + 1e-6 * scale


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_encoder_runs_padded_batches_on_their_valid_tokens(gpu_device, dtype):
    """The stack packs the valid tokens once and runs every layer on them; with the switch off it keeps
    the padded layout (attention in place or gather/scatter per layer).  Same numbers at the valid
    positions, zeros at the padded ones; masks with holes, padding on both sides and an empty row."""
    cfg, m, sd = make(dict(SMALL, attention_type="flash"))
    ids = torch.randint(0, 200, (5, 150), generator=torch.Generator().manual_seed(8))
    for case in ("one run", "holes"):
        mask = torch.ones(5, 150)
        mask[0, :40] = 0
        mask[1, 90:] = 0
        mask[2, :10] = 0
        mask[2, 130:] = 0
        mask[4, :] = 0
        if case == "holes":
            mask[3, 20:25] = 0
        m = m.to(gpu_device).to(dtype)
        dmask = mask.to(gpu_device)
        assert m.encoder.pack_padded_batches
        with torch.no_grad():
            got = m(ids.to(gpu_device), dmask)
            m.encoder.pack_padded_batches = False
            ref = m(ids.to(gpu_device), dmask)
            m.encoder.pack_padded_batches = True
        valid = mask.bool()
        tol = 1e-5 if dtype == torch.float32 else 3e-2
        assert (got.float().cpu()[valid] - ref.float().cpu()[valid]).abs().max().item() <= tol
        assert (got.cpu()[~valid] == 0).all()
        if dtype == torch.float32:
            for b in range(4):
                want = OM.encoder_forward(sd, cfg, ids[b][valid[b]][None])[0]
                assert (got.cpu()[b][valid[b]] - want).abs().max().item() <= 2e-3, (case, b)


def test_packed_stack_is_off_for_decoders_and_sparse_types(gpu_device):
    from turbot5_amd import T5Config, T5EncoderModel, T5Model
    enc = T5EncoderModel(T5Config(**dict(SMALL, attention_type="local", sliding_window=64)))
    assert not enc.encoder.pack_padded_batches
    full = T5Model(T5Config(**dict(SMALL, attention_type="flash")))
    assert full.encoder.pack_padded_batches and not full.decoder.pack_padded_batches


def test_local_encoder_with_right_padding(gpu_device):
    """T5LocalAttention takes right-padded batches (per-sequence key limit in the kernel); other masks raise."""
    cfg, m, sd = make(dict(SMALL, attention_type="local", sliding_window=64))
    ids = torch.randint(0, 200, (3, 256), generator=torch.Generator().manual_seed(9))
    mask = torch.ones(3, 256)
    mask[0, 200:] = 0
    mask[2, 30:] = 0
    want = OM.encoder_forward(sd, cfg, ids, mask, attention_type="local")
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device), mask.to(gpu_device)).cpu()
    valid = mask.bool()
    assert (got[valid] - want[valid]).abs().max().item() <= 2e-3
    # padding on the left, and on both sides: a first row and a length per sequence; positions stay row indices
    left = torch.ones(3, 256)
    left[1, :10] = 0
    left[2, :77] = 0
    left[2, 250:] = 0
    want = OM.encoder_forward(sd, cfg, ids, left, attention_type="local")
    with torch.no_grad():
        got = m(ids.to(gpu_device), left.to(gpu_device)).cpu()
    assert (got[left.bool()] - want[left.bool()]).abs().max().item() <= 2e-3
    holes = torch.ones(3, 256)     # masks with holes: the keys' validity as bit sets
    holes[1, 40:50] = 0
    holes[2, ::7] = 0
    holes[2, :20] = 0
    want = OM.encoder_forward(sd, cfg, ids, holes, attention_type="local")
    with torch.no_grad():
        got = m(ids.to(gpu_device), holes.to(gpu_device)).cpu()
    assert (got[holes.bool()] - want[holes.bool()]).abs().max().item() <= 2e-3


def test_transient_global_encoder_with_right_padding(gpu_device):
    """T5TransientGlobalAttention takes right-padded batches: per-sequence key limit and side-token count
    in the kernels, the side-token producer leaves the padding out."""
    cfg, m, sd = make(dict(SMALL, attention_type="transient-global", sliding_window=64, global_block_size=8))
    ids = torch.randint(0, 200, (3, 256), generator=torch.Generator().manual_seed(10))
    mask = torch.ones(3, 256)
    mask[0, 203:] = 0                # orphan tokens after the last full side block
    mask[2, 30:] = 0
    want = OM.encoder_forward(sd, cfg, ids, mask, attention_type="transient-global")
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device), mask.to(gpu_device)).cpu()
    valid = mask.bool()
    assert (got[valid] - want[valid]).abs().max().item() <= 2e-3
    # padding on the left and on both sides: the reference's block ids for such rows (side tokens before the first
    # token are empty, the last one takes every token from its first row on), first rows inside a side block
    left = torch.ones(3, 256)
    left[0, :19] = 0
    left[1, :64] = 0
    left[1, 201:] = 0
    left[2, :5] = 0
    left[2, 9:] = 0                  # four tokens: no side token at all
    want = OM.encoder_forward(sd, cfg, ids, left, attention_type="transient-global")
    with torch.no_grad():
        got = m(ids.to(gpu_device), left.to(gpu_device)).cpu()
    assert (got[left.bool()] - want[left.bool()]).abs().max().item() <= 2e-3
    # masks with holes: validity bit sets and a side-token count per sequence -- a side block whose END token is
    # masked (its tokens still have their side token while a later END is valid), a masked tail, scattered holes
    holes = torch.ones(3, 256)
    holes[0, 40:50] = 0              # covers the END of side block 5 (row 47)
    holes[0, 250:] = 0
    holes[1, ::7] = 0
    holes[1, :20] = 0
    holes[2, 100:180] = 0
    holes[2, 255] = 0                # the last END: rows 248..254 join side token 30
    want = OM.encoder_forward(sd, cfg, ids, holes, attention_type="transient-global")
    with torch.no_grad():
        got = m(ids.to(gpu_device), holes.to(gpu_device)).cpu()
    assert (got[holes.bool()] - want[holes.bool()]).abs().max().item() <= 2e-3


def test_block_encoder_with_right_padding(gpu_device):
    """T5BlockAttention on right-padded batches: the reference's additive mask as it lies over the key list
    [global tokens | own block] (its layout quirk included), global rows seeing every key."""
    cfg, m, sd = make(dict(SMALL, attention_type="block", sliding_window=64, global_block_size=16))
    ids = torch.randint(0, 200, (4, 256), generator=torch.Generator().manual_seed(11))
    mask = torch.ones(4, 256)
    mask[0, 200:] = 0                # inside the last block, past its first 16 columns
    mask[1, 70:] = 0                 # inside the second block, within its first 16 columns
    mask[2, 30:] = 0                 # inside block 0
    mask[3, 128:] = 0                # exactly at a block boundary
    want = OM.encoder_forward(sd, cfg, ids, mask, attention_type="block")
    m = m.to(gpu_device)
    with torch.no_grad():
        got = m(ids.to(gpu_device), mask.to(gpu_device)).cpu()
    valid = mask.bool()
    assert (got[valid] - want[valid]).abs().max().item() <= 2e-3
    other = torch.ones(4, 256)     # left padding and holes: validity bit sets
    other[1, :10] = 0
    other[2, 100:140] = 0
    other[3, ::5] = 0
    want = OM.encoder_forward(sd, cfg, ids, other, attention_type="block")
    with torch.no_grad():
        got = m(ids.to(gpu_device), other.to(gpu_device)).cpu()
    valid = other.bool()
    assert (got[valid] - want[valid]).abs().max().item() <= 2e-3


@pytest.mark.parametrize("attention_dtype", [None, torch.bfloat16])
def test_graphed_greedy_decode_equals_eager(gpu_device, attention_dtype):
    """One HIP graph per decoding step (static KV cache, key length read from device memory).  The graph is
    captured once and replayed for every step of every later call: three memories, eager decoding and
    synchronisations in between, every call checked against the eager loop (tokens, and logits to rounding)."""
    from turbot5_amd import T5Config, T5Model
    torch.manual_seed(0)
    cfg = T5Config(**dict(SMALL, attention_type="flash", attention_dtype=attention_dtype))
    m = T5Model(cfg).eval().to(gpu_device)
    steps = 10
    for trial in range(3):
        mem = torch.randn(3, 600, 128, generator=torch.Generator().manual_seed(trial)).to(gpu_device)
        want = m.greedy_decode(encoder_outputs=mem, max_new_tokens=steps)
        torch.cuda.synchronize()
        got, logits = m.greedy_decode_graphed(mem, steps, return_logits=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want), trial
        # logits of the eager pass over the same tokens (teacher forcing through the full decoder)
        dec_in = torch.cat([torch.full((3, 1), cfg.decoder_start_token_id, device=gpu_device), want[:, :-1]], dim=1)
        with torch.no_grad():
            ref = m(None, dec_in, encoder_outputs=mem)[0]
        tol = 2e-3 if attention_dtype is None else 6e-2
        assert (logits - ref.float()).abs().max().item() <= tol * max(1.0, ref.abs().max().item())
    assert len(m._decode_graphs) == 1          # one capture served all three calls
    graph = next(iter(m._decode_graphs.values()))["graph"]
    m.to(torch.float32 if attention_dtype is None else torch.float32)      # same dtype: parameters stay where they are
    m.greedy_decode_graphed(mem, steps)
    assert next(iter(m._decode_graphs.values()))["graph"] is graph
    m.lm_head.weight = torch.nn.Parameter(m.lm_head.weight.detach().clone())   # a parameter that moved: capture again
    got = m.greedy_decode_graphed(mem, steps)
    assert next(iter(m._decode_graphs.values()))["graph"] is not graph
    assert torch.equal(got, m.greedy_decode(encoder_outputs=mem, max_new_tokens=steps))


@pytest.mark.parametrize("attention_type,extra", [("flash", {}), ("local", dict(sliding_window=64)),
                                                  ("transient-global", dict(sliding_window=64, global_block_size=8))])
def test_encoder_forward_as_one_graph(gpu_device, attention_type, extra):
    """A fixed-shape encoder pass captured once and replayed: several inputs, eager passes and
    synchronisations in between, every replay checked against the eager result."""
    from turbot5_amd import GraphedForward
    cfg, m, sd = make(dict(SMALL, attention_type=attention_type, **extra))
    m = m.to(gpu_device)
    ids = torch.randint(0, 200, (2, 256), generator=torch.Generator().manual_seed(11)).to(gpu_device)
    graphed = GraphedForward(m, ids)
    for trial in range(4):
        ids = torch.randint(0, 200, (2, 256), generator=torch.Generator().manual_seed(20 + trial)).to(gpu_device)
        with torch.no_grad():
            want = m(ids)
        torch.cuda.synchronize()
        got = graphed(ids)
        torch.cuda.synchronize()
        assert (got - want).abs().max().item() <= 1e-5, trial
    with pytest.raises(ValueError):
        graphed(ids[:, :100])
    with pytest.raises(ValueError):
        graphed(ids, None)
    if attention_type == "flash":      # a mask keeps the pattern it was captured with
        mask = torch.ones(2, 256, device=gpu_device)
        mask[1, 200:] = 0
        masked = GraphedForward(m, ids, mask)
        with torch.no_grad():
            want = m(ids, mask)
        assert (masked(ids, mask.clone()) - want).abs().max().item() <= 1e-5
        other = mask.clone()
        other[1, 150:] = 0
        with pytest.raises(ValueError):
            masked(ids, other)


def test_graphed_greedy_decode_over_padded_memories(gpu_device):
    """Encoder memories of different lengths: the captured step reads each memory's first row and length
    from device buffers, so one graph serves masks of the same shape with other lengths."""
    from turbot5_amd import T5Config, T5Model
    torch.manual_seed(1)
    m = T5Model(T5Config(**dict(SMALL, attention_type="flash"))).eval().to(gpu_device)
    steps = 8
    for trial, lens in enumerate(([600, 17, 333], [5, 600, 128], [600, 600, 599])):
        mem = torch.randn(3, 600, 128, generator=torch.Generator().manual_seed(30 + trial)).to(gpu_device)
        mask = (torch.arange(600)[None, :] < torch.tensor(lens)[:, None]).float().to(gpu_device)
        if trial == 1:
            mask = mask.flip(1)          # left padding
        want = m.greedy_decode(encoder_outputs=mem, attention_mask=mask, max_new_tokens=steps)
        torch.cuda.synchronize()
        got = m.greedy_decode_graphed(mem, steps, attention_mask=mask)
        torch.cuda.synchronize()
        assert torch.equal(got, want), trial
    assert len(m._decode_graphs) == 1
    holes = torch.ones(3, 600, device=gpu_device)
    holes[0, 10:20] = 0
    with pytest.raises(NotImplementedError):
        m.greedy_decode_graphed(mem, steps, attention_mask=holes)
